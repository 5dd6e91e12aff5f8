"""Parity of the fp16 x int4 MFMA GEMM (M > 16) and its fused prologue/epilogues against the CPU oracle.

Tolerance: max|y - y_ref| <= 1e-2 * RMS(y_ref) (stated by the task for the fp16 x int4 path).
Full-size shapes are checked on a sample of output columns (the oracle GEMM of the whole matrix would
take minutes on the host), plus size-independent properties.
"""
import numpy as np
import pytest

import oracle
from nnfusion_amd import datagen

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _t(gpu, *arrays):
    import torch

    return [None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(gpu) for a in arrays]


def _rms(x):
    return float(np.sqrt(np.mean(np.asarray(x, np.float64) ** 2)))


def _check(y, ref, tol=TOL):
    err = float(np.abs(y.astype(np.float32) - ref.astype(np.float32)).max())
    rms = _rms(ref)
    assert err <= tol * max(rms, 1e-6), (err, rms)


# Plans of the MFMA tile GEMM, passed per call through nnf_w4a16_gemm_variant / nnf_w4a16_gemm_fused_variant (struct
# nnf_plan): None = the library's own choice of kernel and plan; otherwise (tile_rows, k_parts[, tile_cols]): tiles of
# 256, 128, 64 or 32 rows by 256 columns (128 where given: products without SiLU-gate), and the number of workgroups that
# share a tile (each a part of K; parts parked in the workspace and added by the second launch)
PLANS = [None, (256, 1, 256), (256, 2, 256), (128, 1, 256), (128, 3, 256), (64, 1, 256), (64, 2, 256), (32, 1), (32, 3),
         (256, 1, 128), (256, 3, 128), (128, 1, 128), (128, 2, 128), (64, 1, 128), (64, 3, 128)]


@pytest.fixture(params=PLANS, ids=lambda p: "auto" if p is None else "rows%d-parts%d" % p[:2] + ("-cols%d" % p[2] if len(p) > 2 else ""))
def plan(request):
    """Keyword arguments for ops.w4a16_gemm_fused / _gemm below."""
    return {} if request.param is None else {"variant": "gemm_mfma", "plan": request.param}


def _gemm(ta, tw, ts, plan_kw, workspace=None):
    from nnfusion_amd import ops

    if plan_kw:
        return ops.w4a16_gemm_variant(ta, tw, ts, plan_kw["variant"], plan=plan_kw["plan"], workspace=workspace)
    return ops.w4a16_gemm(ta, tw, ts, workspace=workspace)


def _big_ws(gpu):
    import torch

    return torch.empty(64 << 20, dtype=torch.uint8, device=gpu)


@pytest.mark.parametrize("m,n,k", [(200, 300, 1024), (64, 520, 2048), (130, 128, 512), (17, 40, 1280)])
def test_gemm_every_tile_plan_matches_oracle(gpu, plan, m, n, k):
    import torch

    from nnfusion_amd import ops

    print(f"case plan={plan} M={m} N={n} K={k}", flush=True)
    a, wq, s = datagen.w4a16_case(2, m, n, k)
    ta, tw, ts = _t(gpu, a, wq, s)
    y = _gemm(ta, tw, ts, plan, workspace=_big_ws(gpu))
    torch.cuda.synchronize()
    _check(y.cpu().numpy(), oracle.w4a16_gemm(a, wq, s, f32_out=True))


@pytest.mark.parametrize("m,n,k", [
    (128, 256, 128), (256, 256, 256), (17, 32, 128), (100, 96, 384), (300, 520, 1024),
    (512, 1024, 2048), (257, 33, 512), (1024, 512, 4096), (2048, 2048, 512),
])
def test_gemm_matches_oracle(gpu, m, n, k):
    import torch

    from nnfusion_amd import ops

    print(f"case M={m} N={n} K={k}", flush=True)
    a, wq, s = datagen.w4a16_case(0, m, n, k)
    ta, tw, ts = _t(gpu, a, wq, s)
    y = ops.w4a16_gemm(ta, tw, ts)
    torch.cuda.synchronize()
    ref = oracle.w4a16_gemm(a, wq, s, f32_out=True)
    _check(y.cpu().numpy(), ref)


def _random_shapes(count):
    rng = np.random.default_rng(777)
    out = []
    for _ in range(count):
        m = int(rng.choice([1, 2, 3, 8, 15, 16, 17, 31, 32, 33, 40, 41, 64, 65, 127, 128, 129, 200, 256, 300, 513]))
        n = int(rng.choice([1, 15, 16, 17, 64, 100, 255, 256, 257, 500, 1000, 1024, 2000, 4096, 5000]))
        k = int(rng.choice([128, 256, 384, 512, 640, 1024, 1152, 2048, 2560, 3072, 4096, 5120, 6144, 7168, 8192, 11008, 14336]))
        if m * n * k > 300 * 2000 * 4096:
            n = 256
        out.append((m, n, k, int(rng.integers(0, 16))))
    return out


@pytest.mark.parametrize("m,n,k,zp", _random_shapes(150))
def test_gemm_random_shapes(gpu, m, n, k, zp):
    """Shapes drawn across the routes of nnf_w4a16_gemm (the row-streaming kernels with a fixed and a run-time K, ranges of
    K, the MFMA GEMV, stream-K tiles of every height), every zero point."""
    import torch

    from nnfusion_amd import ops

    a, wq, s = datagen.w4a16_case(m + 5 * n + 11 * k + zp, m, n, k)
    ta, tw, ts = _t(gpu, a, wq, s)
    y = ops.w4a16_gemm(ta, tw, ts, zp=zp)
    torch.cuda.synchronize()
    ref = oracle.w4a16_gemm(a, wq, s, zp=zp, f32_out=True)
    _check(y.cpu().numpy(), ref)


@pytest.mark.parametrize("m", [1, 5, 16])
def test_gemm_kernel_serves_small_m(gpu, m):
    """The tile GEMM asked for by variant (the library's own choice for these shapes is a GEMV kernel)."""
    import torch

    from nnfusion_amd import ops

    a, wq, s = datagen.w4a16_case(4, m, 320, 512)
    ta, tw, ts = _t(gpu, a, wq, s)
    y = ops.w4a16_gemm_variant(ta, tw, ts, "gemm_mfma", workspace=_big_ws(gpu))
    torch.cuda.synchronize()
    _check(y.cpu().numpy(), oracle.w4a16_gemm(a, wq, s, f32_out=True))


def test_gemm_one_hot_rows_select_weights(gpu):
    """A = rows of the identity  =>  Y[m, n] = fp16((q[n, m] - 8) * s[n, m/128]) exactly:
    pins nibble order, the K-slot permutation shared by the A and W fragments, and scale indexing."""
    import torch

    from nnfusion_amd import ops

    n, k = 160, 256
    _, wq, s = datagen.w4a16_case(5, 1, n, k)
    a = np.eye(k, dtype=np.float16)
    ta, tw, ts = _t(gpu, a, wq, s)
    y = ops.w4a16_gemm(ta, tw, ts).cpu().numpy()
    torch.cuda.synchronize()
    wd = oracle.dequantize_w4(wq, s)  # [n, k]
    np.testing.assert_array_equal(y, wd.T.astype(np.float16))


@pytest.mark.parametrize("m,n,k", [(16, 8192, 8192), (128, 8192, 8192), (1024, 8192, 8192), (4096, 8192, 8192),
                                   (32, 8192, 8192), (16, 22016, 4096), (16, 4096, 11008),
                                   (250, 21000, 1024), (100, 20004, 768), (640, 8192, 4096), (256, 22016, 4096)])
def test_gemm_full_size_sampled_columns(gpu, m, n, k):
    """configs[2] shapes (and batched-decode shapes on the row-streaming kernels: one launch, over ranges of K; and
    products whose tiles fill at least half of the CUs, which run whole tiles, one workgroup each, with ragged rows
    and columns): all M rows, 192 sampled output columns against the oracle; and linearity in A
    on the whole output (Y(2A) == 2 Y(A) bit for bit, as scaling by 2 is exact outside the subnormal range)."""
    import torch

    from nnfusion_amd import ops

    print(f"case M={m} N={n} K={k}", flush=True)
    a, wq, s = datagen.w4a16_case(0, m, n, k)
    ta, tw, ts = _t(gpu, a, wq, s)
    y = ops.w4a16_gemm(ta, tw, ts)
    torch.cuda.synchronize()
    rng = np.random.default_rng(0)
    cols = np.sort(rng.choice(n, 192, replace=False))
    ref = oracle.w4a16_gemm(a, wq[cols], s[cols], f32_out=True)
    _check(y.cpu().numpy()[:, cols], ref)
    # Scaling by two is exact everywhere except where the fp16 result itself is subnormal (no kernel rescales the
    # activations: the nibbles are decoded to exact fp16 integers on the weight side).
    y1 = ops.w4a16_gemm(ta, tw, ts)
    y2 = ops.w4a16_gemm(ta * 2, tw, ts)
    torch.cuda.synchronize()
    normal = y1.abs() >= 2.0 ** -13
    assert torch.equal(y2[normal], (y1 * 2)[normal])


def test_fused_bias_residual(gpu, plan):
    import torch

    from nnfusion_amd import ops

    m, n, k = 200, 288, 512
    a, wq, s = datagen.w4a16_case(6, m, n, k)
    bias = datagen.normal_f16(6, datagen.S_BIAS, (n,))
    res = datagen.normal_f16(6, datagen.S_RES, (m, n))
    ta, tw, ts, tb, tr = _t(gpu, a, wq, s, bias, res)
    ws = _big_ws(gpu)
    y_b = ops.w4a16_gemm_fused(ta, tw, ts, bias=tb, workspace=ws, **plan).cpu().numpy()
    y_r = ops.w4a16_gemm_fused(ta, tw, ts, residual=tr, workspace=ws, **plan).cpu().numpy()
    y_br = ops.w4a16_gemm_fused(ta, tw, ts, bias=tb, residual=tr, workspace=ws, **plan).cpu().numpy()
    torch.cuda.synchronize()
    d = oracle.w4a16_gemm(a, wq, s)  # fp16 tensor of the unfused Dot
    ref_b = oracle.add_f16(d, np.broadcast_to(bias, (m, n)).copy())
    ref_r = oracle.add_f16(d, res)
    ref_br = oracle.add_f16(ref_b, res)
    _check(y_b, ref_b)
    _check(y_r, ref_r)
    _check(y_br, ref_br)


@pytest.mark.parametrize("m,n,k", [(257, 300, 512), (90, 36, 384), (33, 1001, 256)])
def test_fused_bias_residual_ragged_columns(gpu, plan, m, n, k):
    """N not a multiple of 8 (no 16-byte row pieces), M not a multiple of the tile: the element-wise tail of the
    row-major epilogue, with bias and residual."""
    import torch

    from nnfusion_amd import ops

    a, wq, s = datagen.w4a16_case(13, m, n, k)
    bias = datagen.normal_f16(13, datagen.S_BIAS, (n,))
    res = datagen.normal_f16(13, datagen.S_RES, (m, n))
    ta, tw, ts, tb, tr = _t(gpu, a, wq, s, bias, res)
    ws = _big_ws(gpu)
    y = _gemm(ta, tw, ts, plan, workspace=ws).cpu().numpy()
    y_br = ops.w4a16_gemm_fused(ta, tw, ts, bias=tb, residual=tr, workspace=ws, **plan).cpu().numpy()
    torch.cuda.synchronize()
    d = oracle.w4a16_gemm(a, wq, s)
    _check(y, oracle.w4a16_gemm(a, wq, s, f32_out=True))
    _check(y_br, oracle.add_f16(oracle.add_f16(d, np.broadcast_to(bias, (m, n)).copy()), res))


def test_fused_silu_gate_ragged_columns(gpu, plan):
    import torch

    from nnfusion_amd import ops

    m, n, k = 70, 100, 256
    a, wq, s = datagen.w4a16_case(14, m, 2 * n, k)
    ta, tw, ts = _t(gpu, a, wq, s)
    y = ops.w4a16_gemm_fused(ta, tw, ts, act=1, workspace=_big_ws(gpu), **plan).cpu().numpy()
    torch.cuda.synchronize()
    gu = oracle.w4a16_gemm(a, wq, s)
    ref = oracle.silu_mul_f16(np.ascontiguousarray(gu[:, :n]), np.ascontiguousarray(gu[:, n:]))
    err = np.abs(y.astype(np.float32) - ref.astype(np.float32))
    assert y.shape == (m, n)
    assert _rms(err) <= 1e-3 * _rms(ref) and err.max() <= 5e-2 * max(_rms(ref), 1e-3)


def test_fused_rmsnorm_prologue(gpu, plan):
    import torch

    from nnfusion_amd import ops

    m, n, k = 130, 256, 1024
    a, wq, s = datagen.w4a16_case(7, m, n, k)
    gamma = datagen.normal_f16(7, datagen.S_GAMMA, (k,), 1.0, 0.1)
    ta, tw, ts, tg = _t(gpu, a, wq, s, gamma)
    y = ops.w4a16_gemm_fused(ta, tw, ts, rms_gamma=tg, rms_eps=1e-6, workspace=_big_ws(gpu), **plan).cpu().numpy()
    torch.cuda.synchronize()
    xn = oracle.rmsnorm_f16(a, gamma, 1e-6)
    _check(y, oracle.w4a16_gemm(xn, wq, s, f32_out=True))


def test_fused_silu_gate(gpu, plan):
    import torch

    from nnfusion_amd import ops

    m, n, k = 150, 192, 512  # n = intermediate size; weights hold 2n rows (gate then up)
    a, wq, s = datagen.w4a16_case(8, m, 2 * n, k)
    ta, tw, ts = _t(gpu, a, wq, s)
    y = ops.w4a16_gemm_fused(ta, tw, ts, act=1, workspace=_big_ws(gpu), **plan).cpu().numpy()
    torch.cuda.synchronize()
    gu = oracle.w4a16_gemm(a, wq, s)
    g = np.ascontiguousarray(gu[:, :n])
    u = np.ascontiguousarray(gu[:, n:])
    ref = oracle.silu_mul_f16(g, u)
    assert y.shape == (m, n)
    # The stated tolerance applies to the GEMM outputs g and u: delta = 1e-2 * RMS(gu).  It is
    # carried through h = silu(g) * u element-wise: |dh| <= |dh/dg| delta + |dh/du| delta with
    # |dh/dg| <= 1.1 |u| and |dh/du| = |silu(g)|, plus one fp16 rounding of h.
    delta = TOL * _rms(gu)
    g32, u32 = g.astype(np.float32), u.astype(np.float32)
    silu = g32 / (1.0 + np.exp(-g32))
    bound = delta * (1.1 * np.abs(u32) + np.abs(silu)) + np.abs(ref.astype(np.float32)) * 2.0 ** -10 + 1e-6
    err = np.abs(y.astype(np.float32) - ref.astype(np.float32))
    assert np.all(err <= bound), float((err - bound).max())
    # and the typical error is far smaller: RMS of the error within 1e-3 of RMS(h)
    assert _rms(err) <= 1e-3 * _rms(ref)


@pytest.mark.parametrize("m,n,k", [(1, 320, 1024), (5, 320, 1024), (16, 320, 1024), (2, 520, 4096), (24, 320, 2048), (32, 1000, 4096),
                                   (16, 136, 11008), (24, 264, 8192), (7, 320, 3584)])
def test_fused_small_m_goes_through_the_gemv_kernel(gpu, m, n, k):
    """Decode shapes with a prologue / epilogue: the GEMV kernels (M = 1; 2 .. 32 rows in one launch or over ranges of
    K) multiply the RMSNorm weight in themselves and apply rstd, bias, residual and the gate at their flush (over ranges
    of K: in the reduction pass).  The workspace is the one the query asks for: rstd and partial sums, no M x K
    activations and no M x 2N products."""
    import torch

    from nnfusion_amd import ops

    a, wq, s = datagen.w4a16_case(11, m, 2 * n, k)
    gamma = datagen.normal_f16(11, datagen.S_GAMMA, (k,), 1.0, 0.1)
    bias = datagen.normal_f16(11, datagen.S_BIAS, (n,))
    res = datagen.normal_f16(11, datagen.S_RES, (m, n))
    ta, tw, ts, tg, tb, tr = _t(gpu, a, wq, s, gamma, bias, res)
    xn = oracle.rmsnorm_f16(a, gamma, 1e-6)
    # RMSNorm + bias + residual on the first n weight rows
    y = ops.w4a16_gemm_fused(ta, tw[:n].contiguous(), ts[:n].contiguous(), rms_gamma=tg, rms_eps=1e-6, bias=tb,
                             residual=tr).cpu().numpy()
    d = oracle.w4a16_gemm(xn, wq[:n], s[:n])
    ref = oracle.add_f16(oracle.add_f16(d, np.broadcast_to(bias, (m, n)).copy()), res)
    _check(y, ref)
    # RMSNorm + SiLU gate over all 2n rows (gate rows, then up rows)
    yg = ops.w4a16_gemm_fused(ta, tw, ts, rms_gamma=tg, rms_eps=1e-6, act=1).cpu().numpy()
    torch.cuda.synchronize()
    gu = oracle.w4a16_gemm(xn, wq, s)
    # the bound the tolerance of the two products (delta on each of gate and up) leaves on SiLU(gate) * up
    g, u = np.ascontiguousarray(gu[:, :n]), np.ascontiguousarray(gu[:, n:])
    refg = oracle.silu_mul_f16(g, u).astype(np.float32)
    delta = TOL * _rms(gu)
    g32, u32 = g.astype(np.float32), u.astype(np.float32)
    bound = delta * (1.1 * np.abs(u32) + np.abs(g32 / (1.0 + np.exp(-g32)))) + np.abs(refg) * 2.0 ** -10 + 1e-6
    err = np.abs(yg.astype(np.float32) - refg)
    assert _rms(err) <= 1e-3 * _rms(refg) and np.all(err <= bound), float((err - bound).max())


@pytest.mark.parametrize("m", [3, 24, 200])
def test_residual_may_alias_the_output(gpu, m):
    import torch

    from nnfusion_amd import ops

    n, k = 288, 512
    a, wq, s = datagen.w4a16_case(12, m, n, k)
    res = datagen.normal_f16(12, datagen.S_RES, (m, n))
    ta, tw, ts, tr = _t(gpu, a, wq, s, res)
    y = ops.w4a16_gemm_fused(ta, tw, ts, residual=tr, out=tr, workspace=_big_ws(gpu)).cpu().numpy()
    torch.cuda.synchronize()
    _check(y, oracle.add_f16(oracle.w4a16_gemm(a, wq, s), res))


def test_rejects_bad_arguments(gpu):
    import torch

    from nnfusion_amd import ops

    a, wq, s = datagen.w4a16_case(9, 4, 64, 256)
    ta, tw, ts = _t(gpu, a, wq, s)
    with pytest.raises(ops.NnfError) as e:
        ops.w4a16_gemm(ta, tw, ts, zp=16)
    assert e.value.status == -2
    from nnfusion_amd import _lib

    lib = _lib.kernels()
    y = torch.empty((4, 64), dtype=torch.float16, device=gpu)
    args = (ta.data_ptr(), tw.data_ptr(), ts.data_ptr(), y.data_ptr())
    assert lib.nnf_w4a16_gemm(None, *args, 4, 64, 256, 64, 8, None, 0) == -2      # group != 128
    assert lib.nnf_w4a16_gemm(None, *args, 4, 64, 192, 128, 8, None, 0) == -2     # K % group != 0
    assert lib.nnf_w4a16_gemm(None, *args, 0, 64, 256, 128, 8, None, 0) == -1     # empty M
    assert lib.nnf_w4a16_gemm(None, None, *args[1:], 4, 64, 256, 128, 8, None, 0) == -1  # null pointer
    assert lib.nnf_w4a16_gemm(None, args[0] + 2, *args[1:], 4, 64, 256, 128, 8, None, 0) == -1  # misaligned
    assert b"unsupported" in lib.nnf_status_string(-2)


# ---- the fused parts on the kernels that serve a few rows ------------------------------------------------------------
# auto: the library's choice (one row: the row-streaming GEMV; up to 32 rows: the row-streaming MFMA kernel, over ranges
# of K with the reduction pass where K is long; otherwise the MFMA GEMV kernel with a pre-pass and an element-wise
# kernel); gemv_rows / gemv_mfma: that family only, where it takes the shape.
@pytest.mark.parametrize("variant", ["auto", "gemv_rows", "gemv_mfma"])
@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (1, 300, 1024), (1, 1000, 11008), (3, 304, 2048), (16, 4096, 4096),
                                   (16, 520, 3584), (8, 1000, 11008), (24, 304, 4096), (24, 1000, 8192), (7, 100, 2176)])
def test_fused_parts_with_few_rows(gpu, variant, m, n, k):
    import torch

    from nnfusion_amd import ops

    print(f"case variant={variant} M={m} N={n} K={k}", flush=True)
    a, wq, s = datagen.w4a16_case(21, m, 2 * n, k)  # 2n weight rows: the gate product uses all, the others the first n
    bias = datagen.normal_f16(21, datagen.S_BIAS, (n,))
    res = datagen.normal_f16(21, datagen.S_RES, (m, n))
    gamma = datagen.normal_f16(21, datagen.S_GAMMA, (k,), 1.0, 0.1)
    ta, tw, ts, tb, tr, tg = _t(gpu, a, wq, s, bias, res, gamma)
    tw1, ts1 = tw[:n].contiguous(), ts[:n].contiguous()
    kw = {} if variant == "auto" else {"variant": variant}
    ws = _big_ws(gpu)

    def run(w, sc, **fused):
        try:
            return ops.w4a16_gemm_fused(ta, w, sc, workspace=ws, **fused, **kw)
        except ops.NnfError as e:
            assert e.status == -2 and variant != "auto"  # this family does not take the shape
            return None

    d = oracle.w4a16_gemm(a, wq[:n], s[:n])  # fp16 tensor of the unfused Dot
    ref_b = oracle.add_f16(d, np.broadcast_to(bias, (m, n)).copy())
    y = run(tw1, ts1, bias=tb)
    if y is None:
        pytest.skip("variant does not serve this shape")
    _check(y.cpu().numpy(), ref_b)
    _check(run(tw1, ts1, residual=tr).cpu().numpy(), oracle.add_f16(d, res))
    _check(run(tw1, ts1, bias=tb, residual=tr).cpu().numpy(), oracle.add_f16(ref_b, res))
    # the residual in place: the output buffer holds it
    out = tr.clone()
    y_in_place = ops.w4a16_gemm_fused(ta, tw1, ts1, bias=tb, residual=out, out=out, workspace=ws, **kw)
    _check(y_in_place.cpu().numpy(), oracle.add_f16(ref_b, res))
    # RMSNorm prologue alone and with everything behind it
    xn = oracle.rmsnorm_f16(a, gamma, 1e-6)
    dn32 = oracle.w4a16_gemm(xn, wq[:n], s[:n], f32_out=True)
    _check(run(tw1, ts1, rms_gamma=tg, rms_eps=1e-6).cpu().numpy(), dn32)
    dn = oracle.w4a16_gemm(xn, wq[:n], s[:n])
    ref_nbr = oracle.add_f16(oracle.add_f16(dn, np.broadcast_to(bias, (m, n)).copy()), res)
    _check(run(tw1, ts1, rms_gamma=tg, rms_eps=1e-6, bias=tb, residual=tr).cpu().numpy(), ref_nbr)
    # SiLU-gate, without and with the prologue
    for x, fused in ((a, {}), (xn, {"rms_gamma": tg, "rms_eps": 1e-6})):
        gu = oracle.w4a16_gemm(x, wq, s)
        g, u = np.ascontiguousarray(gu[:, :n]), np.ascontiguousarray(gu[:, n:])
        ref = oracle.silu_mul_f16(g, u)
        yg = run(tw, ts, act=1, **fused).cpu().numpy()
        assert yg.shape == (m, n)
        delta = TOL * _rms(gu)
        g32, u32 = g.astype(np.float32), u.astype(np.float32)
        silu = g32 / (1.0 + np.exp(-g32))
        bound = delta * (1.1 * np.abs(u32) + np.abs(silu)) + np.abs(ref.astype(np.float32)) * 2.0 ** -10 + 1e-6
        err = np.abs(yg.astype(np.float32) - ref.astype(np.float32))
        assert np.all(err <= bound), float((err - bound).max())
    torch.cuda.synchronize()


@pytest.mark.parametrize("m,n,k", [(11, 981, 8192), (16, 4096, 8192), (8, 300, 8192), (12, 9000, 8192), (24, 304, 8192),
                                   (8, 1000, 11008), (3, 520, 4096), (200, 300, 1024), (1, 4096, 4096), (16, 48, 2304)])
def test_fused_parts_in_the_workspace_the_query_asks_for(gpu, m, n, k):
    """nnf_w4a16_gemm_fused_workspace_bytes does not know which of the optional parts a call will use, and the kernels
    that serve them differ (8 .. 16 rows at K = 8192 run over two ranges of K without the RMSNorm prologue, in one launch
    with it): a workspace of exactly that size serves every combination."""
    import torch

    from nnfusion_amd import ops

    a, wq, s = datagen.w4a16_case(23, m, 2 * n, k)
    bias = datagen.normal_f16(23, datagen.S_BIAS, (n,))
    res = datagen.normal_f16(23, datagen.S_RES, (m, n))
    gamma = datagen.normal_f16(23, datagen.S_GAMMA, (k,), 1.0, 0.1)
    ta, tw, ts, tb, tr, tg = _t(gpu, a, wq, s, bias, res, gamma)
    tw1, ts1 = tw[:n].contiguous(), ts[:n].contiguous()
    d = oracle.w4a16_gemm(a, wq[:n], s[:n])
    ref_b = oracle.add_f16(d, np.broadcast_to(bias, (m, n)).copy())
    _check(ops.w4a16_gemm_fused(ta, tw1, ts1, bias=tb).cpu().numpy(), ref_b)
    _check(ops.w4a16_gemm_fused(ta, tw1, ts1, residual=tr).cpu().numpy(), oracle.add_f16(d, res))
    out = tr.clone()
    _check(ops.w4a16_gemm_fused(ta, tw1, ts1, bias=tb, residual=out, out=out).cpu().numpy(), oracle.add_f16(ref_b, res))
    xn = oracle.rmsnorm_f16(a, gamma, 1e-6)
    _check(ops.w4a16_gemm_fused(ta, tw1, ts1, rms_gamma=tg, rms_eps=1e-6).cpu().numpy(),
           oracle.w4a16_gemm(xn, wq[:n], s[:n], f32_out=True))
    dn = oracle.w4a16_gemm(xn, wq[:n], s[:n])
    _check(ops.w4a16_gemm_fused(ta, tw1, ts1, rms_gamma=tg, rms_eps=1e-6, residual=tr).cpu().numpy(), oracle.add_f16(dn, res))
    assert ops.w4a16_gemm_fused(ta, tw, ts, act=1).shape == (m, n)
    assert ops.w4a16_gemm_fused(ta, tw, ts, act=1, rms_gamma=tg, rms_eps=1e-6).shape == (m, n)
    torch.cuda.synchronize()
