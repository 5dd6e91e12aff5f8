"""Parity of nnf_wna16_gemm (4- or 8-bit weights, groups of 32 / 64 / 128, scalar or per-(row, group) zero points; HIP,
through the C ABI) against the CPU oracle.

Tolerance (stated by the task): max|y - y_ref| <= 1e-2 * RMS(y_ref), y_ref = the oracle's fp32-accumulated product with
the weights dequantised as (q - z) * s; a one-hot activation row must return the dequantised weights exactly.
"""
import ctypes

import numpy as np
import pytest

import oracle
from nnfusion_amd import datagen

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _case(seed, m, n, k, bits, group, zp_tensor):
    return datagen.wna16_case(seed, m, n, k, bits, group, zp_tensor)


def _run(gpu, a, wq, s, bits, group, zp, zps):
    import torch

    from nnfusion_amd import ops

    t = [torch.from_numpy(x).to(gpu) for x in (a, wq, s)]
    tz = None if zps is None else torch.from_numpy(zps).to(gpu)
    y = ops.wna16_gemm(*t, bits=bits, group=group, zp=zp, zero_points=tz)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def _check(y, ref):
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    err = float(np.abs(y.astype(np.float32) - ref).max())
    assert np.isfinite(y).all()
    assert err <= TOL * max(rms, 1e-6), (err, rms)


SHAPES = [
    # the wavefront-per-row kernel (M <= 16): one row, ragged N, K shorter than one pass of a wavefront, an odd number
    # of groups, the benchmark's shapes
    (1, 4096, 4096), (1, 33, 128), (3, 1000, 512), (16, 257, 2048), (5, 64, 160), (1, 12288, 4096), (8, 300, 11008),
    (16, 4111, 4096), (2, 7, 384),
    # one row, K a multiple of 256: the row-streaming kernel (one, two and three loads per row and
    # wavefront; one, two and four wavefronts per row; fewer rows than wavefronts)
    (1, 300, 1024), (1, 22016, 4096), (1, 4096, 11008), (1, 1000, 8192), (1, 5000, 16384), (1, 257, 2560), (1, 5, 4096),
    # a few rows of 4-bit weights with K = 2048 / 4096 / 8192: the row-streaming MFMA kernel (one, two and four loads per
    # step and wavefront; fewer tiles than CUs, a ragged last tile, several tiles per workgroup)
    (2, 4096, 4096), (5, 300, 2048), (8, 1000, 8192), (16, 48, 8192), (13, 12288, 4096), (16, 9000, 2048),
    (17, 4096, 4096), (32, 1000, 2048), (25, 12288, 4096), (31, 40, 4096),
    # ... with any other K that is a multiple of 256: one piece up to 8192 (two, three, four blocks of 128 per wavefront and
    # step; wavefronts past the end of K), ranges of K above (11008: three; 14336: four; 28672: seven)
    (4, 4096, 3584), (16, 1000, 5120), (9, 300, 7168), (2, 4096, 11008), (16, 4096, 11008), (8, 520, 14336), (5, 64, 28672),
    (16, 33, 2560),
    # the tile kernel: one partial tile, ragged M and N, many tiles, a long K
    (17, 33, 128), (64, 64, 512), (100, 1000, 160), (300, 257, 2048), (128, 4096, 4096), (33, 520, 11008), (1024, 130, 384),
    # 4-bit weights above 16 rows with K a multiple of 256: the stream-K tile GEMM (tiles of 32 x 256, 64 x 128, 128 x 128,
    # 256 x 128, 256 x 256; tiles shared between workgroups and not; ragged M and N)
    (17, 300, 256), (40, 1000, 1024), (100, 257, 2048), (130, 4096, 4096), (700, 3000, 1280), (1100, 2050, 768),
    (1600, 520, 2560), (2000, 8192, 512), (30, 22016, 4096),
    # 8-bit weights above 32 rows (16 at K = 8192): two or three blocks of rows through the row-streaming kernel (two
    # above N = 8192), the last block of one, two and all rows; one block more: the tile kernel
    (33, 4096, 4096), (65, 1000, 2048), (96, 520, 4096), (97, 520, 4096), (48, 300, 8192), (49, 300, 8192), (50, 4111, 4096),
    (64, 9000, 2048), (65, 9000, 2048),
    # enough 128 x 128 tiles to fill the chip: the larger tile kernel; ragged M and N, an odd number of groups
    (2048, 2048, 512), (1100, 4100, 160), (4096, 1030, 384),
    # ... 256 x 128 tiles (one round of them beats two of 128 x 128), 256 x 256 tiles (they fill the chip): ragged M and N
    (1000, 8100, 384), (1990, 8100, 160), (300, 22016, 128),
]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("bits,group,zp_tensor", [
    (4, 32, False), (4, 32, True), (4, 64, False), (4, 64, True), (4, 128, True),
    (8, 32, False), (8, 32, True), (8, 64, True), (8, 128, False), (8, 128, True),
])
def test_wna16_matches_oracle(gpu, m, n, k, bits, group, zp_tensor):
    if k % group:
        pytest.skip("K is not a multiple of the group")
    a, wq, s, zps = _case(m * 131 + n + k + bits + group, m, n, k, bits, group, zp_tensor)
    zp = 7 if bits == 4 else 131
    ref = oracle.wna16_gemm(a, wq, s, bits, group, zp=zp, zero_points=zps, f32_out=True)
    _check(_run(gpu, a, wq, s, bits, group, zp, zps), ref)


@pytest.mark.parametrize("m,n,k", [(4, 70, 640), (40, 70, 640), (2000, 2100, 640), (40, 300, 1024), (300, 520, 768),
                                   (2000, 2100, 512), (1990, 8100, 640)])
@pytest.mark.parametrize("bits,group,zp_tensor", [(4, 32, True), (4, 64, False), (8, 64, True), (8, 128, False), (8, 32, True),
                                                   (4, 64, True), (4, 128, True), (4, 32, False)])
def test_one_hot_rows_return_the_dequantised_weights(gpu, m, n, k, bits, group, zp_tensor):
    """A = e_k: 1 * w is exact in every kernel (m = 2000: the 256 x 128 tiles, m = 1990: the 256 x 256 tiles; K a multiple
    of 256 with 4-bit weights: the stream-K tile GEMM), so the output is fp16((q - z) * s) bit for bit; pins nibble and byte order of weights and zero
    points and the block each scale belongs to, on the device."""
    _, wq, s, zps = _case(5, m, n, k, bits, group, zp_tensor)
    zp = 3 if bits == 4 else 200
    wd = oracle.dequantize_wn(wq, s, bits, group, zp=zp, zero_points=zps)
    ks = [0, 1, 7, 8, 31, 32, 63, 64, 127, 128, 255, 256, 511, 512, 639][:m] if m <= 16 else [(7 * r) % k for r in range(min(m, k))]
    a = np.zeros((m, k), np.float16)
    for r, kk in enumerate(ks):
        a[r, kk] = 1.0
    y = _run(gpu, a, wq, s, bits, group, zp, zps)
    for r, kk in enumerate(ks):
        np.testing.assert_array_equal(y[r], wd[:, kk].astype(np.float16))
    assert not y[len(ks):].any()


@pytest.mark.parametrize("m,k", [(1, 1024), (1, 4096), (1, 11008), (1, 16384), (7, 2048), (16, 4096), (3, 8192), (32, 4096),
                                 (20, 2048), (16, 11008), (6, 5120), (11, 7168), (16, 3584)])
@pytest.mark.parametrize("group,zp_tensor", [(32, True), (64, True), (128, True), (32, False), (64, False)])
def test_one_hot_rows_through_the_row_streaming_kernels(gpu, m, k, group, zp_tensor):
    """4-bit weights with one row and K a multiple of 256, or a few rows and K = 2048 / 4096 / 8192, run on the
    row-streaming kernels: the same pin for their scales and zero points (first and last weight of a group, of a
    wavefront's load, of a wavefront's K segment, of a step, of the row)."""
    n = 700
    _, wq, s, zps = _case(11, 1, n, k, 4, group, zp_tensor)
    wd = oracle.dequantize_wn(wq, s, 4, group, zp=5, zero_points=zps)
    kks = [kk for kk in sorted({0, 1, 31, 32, 63, 64, 127, 128, 255, 256, 511, 512, 1023, 1024, 2047, 2048, 4095, 4096, 6143,
                                6144, 8191, 8192, k // 2 - 1, k // 2, k - 129, k - 33, k - 1}) if kk < k]
    for c in range(0, len(kks), m):
        chunk = kks[c:c + m]
        a = np.zeros((m, k), np.float16)
        for r, kk in enumerate(chunk):
            a[r, kk] = 1.0
        y = _run(gpu, a, wq, s, 4, group, 5, zps)
        for r, kk in enumerate(chunk):
            np.testing.assert_array_equal(y[r], wd[:, kk].astype(np.float16), err_msg="k = %d" % kk)
        assert not y[len(chunk):].any()


@pytest.mark.parametrize("m,k", [(1, 1024), (1, 2048), (1, 2560), (1, 4096), (1, 8192), (1, 11008), (1, 16384), (16, 2048), (7, 4096),
                                 (16, 4096), (3, 8192), (16, 8192), (20, 2048), (32, 4096), (33, 2048), (40, 4096), (24, 8192)])
@pytest.mark.parametrize("group,zp_tensor", [(32, True), (64, True), (128, True), (32, False), (128, False)])
def test_one_hot_rows_through_the_row_streaming_kernels_with_8_bit_weights(gpu, m, k, group, zp_tensor):
    """8-bit weights with one row and K a multiple of 256, or 2 .. 16 rows and K = 2048 / 4096 / 8192 (up to 32 rows at
    2048 / 4096, and a few blocks of that many rows one after the other), run on the
    row-streaming kernels as well (a row is K bytes, a lane meets 16 weights per load): the same pin (first and last
    weight of a group, of a lane, of a wavefront's load, of a wavefront's K segment, of a step, of the row)."""
    n = 700
    _, wq, s, zps = _case(13, 1, n, k, 8, group, zp_tensor)
    wd = oracle.dequantize_wn(wq, s, 8, group, zp=201, zero_points=zps)
    kks = [kk for kk in sorted({0, 1, 15, 16, 31, 32, 63, 64, 127, 128, 255, 256, 511, 512, 1023, 1024, 2047, 2048, 3071, 3072,
                                4095, 4096, 6143, 6144, 8191, 8192, k // 2 - 1, k // 2, k - 129, k - 33, k - 17, k - 1}) if kk < k]
    for c in range(0, len(kks), m):
        chunk = kks[c:c + m]
        a = np.zeros((m, k), np.float16)
        for r, kk in enumerate(chunk):
            a[r, kk] = 1.0
        y = _run(gpu, a, wq, s, 8, group, 201, zps)
        for r, kk in enumerate(chunk):
            np.testing.assert_array_equal(y[r], wd[:, kk].astype(np.float16), err_msg="k = %d" % kk)
        assert not y[len(chunk):].any()


def _random_shapes(count):
    rng = np.random.default_rng(20240607)
    ks = [128, 256, 384, 512, 768, 1024, 1280, 2048, 2560, 3584, 4096, 5120, 7168, 8192, 11008, 14336]
    out = []
    for i in range(count):
        m = int(rng.choice([1, 1, 2, 3, 7, 8, 15, 16, 17, 24, 32, 33, 63, 64, 100, 129, 257, 300]))
        n = int(rng.choice([16, 17, 31, 33, 64, 100, 255, 256, 257, 500, 1000, 1024, 2000, 4096]))
        k = int(rng.choice(ks))
        if m * n * k > 300 * 2000 * 4096:
            n = 256
        out.append((m, n, k, int(rng.choice([4, 4, 4, 8])), int(rng.choice([32, 64, 128])), bool(rng.integers(0, 2)), int(rng.integers(0, 16))))
    return out


@pytest.mark.parametrize("m,n,k,bits,group,zp_tensor,zp", _random_shapes(120))
def test_wna16_random_shapes(gpu, m, n, k, bits, group, zp_tensor, zp):
    """Shapes drawn across the routes of nnf_wna16_gemm (row-streaming kernels with a fixed and a run-time K, ranges of K,
    stream-K tiles, plain kernels), every block parameter and zero point."""
    a, wq, s, zps = _case(m + 3 * n + 7 * k + bits + group, m, n, k, bits, group, zp_tensor)
    zp = zp if bits == 4 else 16 * zp + 3
    ref = oracle.wna16_gemm(a, wq, s, bits, group, zp=zp, zero_points=zps, f32_out=True)
    _check(_run(gpu, a, wq, s, bits, group, zp, zps), ref)


def test_tile_gemm_without_its_workspace_runs_on_the_plain_kernel(gpu):
    """Above 16 rows 4-bit weights want the stream-K tile GEMM's workspace; a caller that brings none (or too little)
    gets the same product from the plain tile kernel."""
    import torch

    from nnfusion_amd import ops

    m, n, k, group = 130, 1024, 4096, 64
    a, wq, s, zps = _case(21, m, n, k, 4, group, True)
    need = ops.wna16_workspace_bytes(m, n, k, 4, group)
    assert need > 0
    t = [torch.from_numpy(x).to(gpu) for x in (a, wq, s, zps)]
    ref = oracle.wna16_gemm(a, wq, s, 4, group, zero_points=zps, f32_out=True)
    for ws_bytes in (need, need - 16, 16):
        y = ops.wna16_gemm(t[0], t[1], t[2], bits=4, group=group, zero_points=t[3],
                           workspace=torch.empty(ws_bytes, dtype=torch.uint8, device=gpu))
        torch.cuda.synchronize()
        _check(y.cpu().numpy(), ref)


def test_default_parameters_are_the_specialised_kernels(gpu):
    import torch

    from nnfusion_amd import ops

    for m, n, k in ((1, 4096, 4096), (16, 1000, 2048), (128, 512, 4096)):
        a, wq, s = datagen.w4a16_case(3, m, n, k)
        t = [torch.from_numpy(x).to(gpu) for x in (a, wq, s)]
        y0 = ops.w4a16_gemm(*t, zp=8)
        y1 = ops.wna16_gemm(*t, bits=4, group=128, zp=8)
        assert torch.equal(y0, y1)
        # ... and a zero-point tensor holding the scalar everywhere takes the plain kernels to the same product
        zps = torch.full((n, (k // 128 + 1) // 2), 0x88, dtype=torch.uint8, device=gpu)
        y2 = ops.wna16_gemm(*t, bits=4, group=128, zero_points=zps)
        torch.cuda.synchronize()
        ref = oracle.wna16_gemm(a, wq, s, 4, 128, zp=8, f32_out=True)
        _check(y2.cpu().numpy(), ref)


def test_wna16_argument_errors(gpu):
    import torch

    from nnfusion_amd import _lib
    from nnfusion_amd.ops import NnfQuant

    lib = _lib.kernels()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device=gpu)
    p = buf.data_ptr()

    def call(q, m=4, n=64, k=256, a=p):
        qp = None if q is None else ctypes.cast(ctypes.pointer(q), ctypes.c_void_p)
        return lib.nnf_wna16_gemm(None, a, p, p, p, m, n, k, qp, None, 0)

    assert call(None) == -1
    assert call(NnfQuant(4, 64, 8, None), a=None) == -1
    assert call(NnfQuant(4, 64, 8, None), a=p + 2) == -1
    assert call(NnfQuant(4, 64, 8, None), m=0) == -1
    assert call(NnfQuant(3, 64, 8, None)) == -2      # bits
    assert call(NnfQuant(4, 16, 8, None)) == -2      # group
    assert call(NnfQuant(4, 64, 16, None)) == -2     # zero point outside 4 bits
    assert call(NnfQuant(8, 64, 256, None)) == -2    # ... outside 8 bits
    assert call(NnfQuant(8, 128, 0, None), k=192) == -2  # K % group
    assert call(NnfQuant(8, 64, 255, None)) == 0
    torch.cuda.synchronize()
