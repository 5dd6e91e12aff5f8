"""The nodes around a quantized product as kernels of their own (RMSNorm, Add, Multiply, Sigmoid, Swish, Dequantize) and the
fused product / MLP block for the block parameters that run them one after the other (nnf_wna16_gemm_fused,
nnf_fused_mlp_wna16), against the CPU oracle.

Bit-exact where the arithmetic is exact in fp32 (Add, Multiply, Dequantize, the bias / residual epilogues); RMSNorm and
the sigmoid go through rsqrt / exp, whose device versions differ from libm's in the last fp32 bit: one fp16 ulp there.
The products: max|y - y_ref| <= 1e-2 * RMS(y_ref), the tolerance of the fp16 x int4 path.
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


def _ulps(y, ref):
    """Largest distance in fp16 steps between two fp16 arrays (finite values of one sign per pair)."""
    a = y.view(np.int16).astype(np.int32)
    b = ref.view(np.int16).astype(np.int32)
    return int(np.abs(a - b).max())


def _check(y, ref, tol=TOL):
    err = float(np.abs(y.astype(np.float32) - ref.astype(np.float32)).max())
    assert err <= tol * max(_rms(ref), 1e-6), (err, _rms(ref))


@pytest.mark.parametrize("rows,cols", [(1, 8), (3, 100), (16, 4096), (256, 11008), (5, 7)])
def test_elementwise_nodes(gpu, rows, cols):
    import torch

    from nnfusion_amd import ops

    rng = np.random.default_rng(rows * 31 + cols)
    a = rng.standard_normal((rows, cols)).astype(np.float16)
    b = rng.standard_normal((rows, cols)).astype(np.float16)
    row = rng.standard_normal(cols).astype(np.float16)
    ta, tb, trow = _t(gpu, a, b, row)
    f = np.float32
    # exact in fp32, one rounding: bit for bit
    assert np.array_equal(ops.elementwise("add", ta, tb).cpu().numpy(), (a.astype(f) + b.astype(f)).astype(np.float16))
    assert np.array_equal(ops.elementwise("add", ta, tb).cpu().numpy(), oracle.add_f16(a, b))
    assert np.array_equal(ops.elementwise("multiply", ta, tb).cpu().numpy(), (a.astype(f) * b.astype(f)).astype(np.float16))
    assert np.array_equal(ops.elementwise("add", ta, trow).cpu().numpy(), (a.astype(f) + row.astype(f)[None, :]).astype(np.float16))
    assert np.array_equal(ops.elementwise("multiply", ta, trow).cpu().numpy(), (a.astype(f) * row.astype(f)[None, :]).astype(np.float16))
    # sigmoid as the reference writes it, 1 / (1 + exp(-x)), in fp64 then rounded: within one fp16 step
    sig = (1.0 / (1.0 + np.exp(-a.astype(np.float64)))).astype(np.float16)
    assert _ulps(ops.elementwise("sigmoid", ta).cpu().numpy(), sig) <= 1
    sw = (a.astype(np.float64) / (1.0 + np.exp(-a.astype(np.float64)))).astype(np.float16)
    assert _ulps(ops.elementwise("swish", ta).cpu().numpy(), sw) <= 1
    # in place
    out = ta.clone()
    ops.elementwise("add", out, tb, out=out)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), oracle.add_f16(a, b))
    # Multiply(x, Sigmoid(x)) as two nodes is the oracle's SiLU * 1
    one = np.ones_like(a)
    two_nodes = ops.elementwise("multiply", ta, ops.elementwise("sigmoid", ta)).cpu().numpy()
    assert _ulps(two_nodes, oracle.silu_mul_f16(a, one)) <= 2


@pytest.mark.parametrize("m,k", [(1, 128), (7, 4096), (40, 11008), (256, 4096), (3, 20000)])
def test_rms_norm_node(gpu, m, k):
    from nnfusion_amd import ops

    rng = np.random.default_rng(m + k)
    x = rng.standard_normal((m, k)).astype(np.float16)
    gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float16)
    tx, tg = _t(gpu, x, gamma)
    y = ops.rms_norm(tx, tg, 1e-6).cpu().numpy()
    assert _ulps(y, oracle.rmsnorm_f16(x, gamma, 1e-6)) <= 1
    # a constant row: x * rsqrt(x^2) * gamma = sign(x) * gamma
    c = np.full((2, k), -3.0, np.float16)
    tc, = _t(gpu, c)
    assert _ulps(ops.rms_norm(tc, tg, 0.0).cpu().numpy(), np.broadcast_to(-gamma, (2, k)).copy()) <= 1


@pytest.mark.parametrize("bits,group,zpt", [(4, 128, False), (4, 32, True), (4, 64, False), (8, 64, True), (8, 128, False)])
@pytest.mark.parametrize("n,k", [(16, 256), (100, 1024), (4096, 4096)])
def test_dequantize_node_is_exact(gpu, bits, group, zpt, n, k):
    from nnfusion_amd import ops

    _, wq, s, z = datagen.wna16_case(n + k, 1, n, k, bits, group, zpt)
    zp = 1 << (bits - 1)
    tw, ts, tz = _t(gpu, wq, s, z if zpt else None)
    w = ops.dequantize(tw, ts, bits=bits, group=group, zp=zp, zero_points=tz).cpu().numpy()
    ref = oracle.dequantize_wn(wq, s, bits, group, zp=zp, zero_points=z if zpt else None)  # fp32, exact products
    assert np.array_equal(w.view(np.uint16), ref.astype(np.float16).view(np.uint16))


def _check_gate(y, gu, n):
    """SiLU(gate) * up against the oracle's, with the bound that the tolerance of the two products (delta on each of gate
    and up) leaves on it: |d(silu(g) u)| <= delta (1.1 |u| + |silu(g)|), plus a rounding step of the result."""
    g, u = np.ascontiguousarray(gu[:, :n]), np.ascontiguousarray(gu[:, n:])
    ref = oracle.silu_mul_f16(g, u).astype(np.float32)
    delta = TOL * _rms(gu)
    g32, u32 = g.astype(np.float32), u.astype(np.float32)
    silu = g32 / (1.0 + np.exp(-g32))
    bound = delta * (1.1 * np.abs(u32) + np.abs(silu)) + np.abs(ref) * 2.0 ** -10 + 1e-6
    err = np.abs(y.astype(np.float32) - ref)
    assert np.all(err <= bound), float((err - bound).max())


Q_CASES = [(4, 32, True), (4, 64, False), (4, 128, True), (8, 128, False), (8, 32, True)]


def _q_ref(a, wq, s, bits, group, zp, z):
    return oracle.wna16_gemm(a, wq, s, bits, group, zp=zp, zero_points=z)  # fp16, the product node's output


@pytest.mark.parametrize("bits,group,zpt", Q_CASES)
@pytest.mark.parametrize("m,n,k", [(1, 512, 1024), (8, 256, 2048), (40, 384, 1024), (200, 256, 512)])
@pytest.mark.parametrize("fused", ["rms", "bias+residual", "residual-in-place", "rms+gate", "gate"])
def test_fused_product_with_other_block_parameters(gpu, fused, m, n, k, bits, group, zpt):
    """nnf_wna16_gemm_fused against the nodes of the unfused graph on the oracle, fp16 tensors between them."""
    import torch

    from nnfusion_amd import ops

    gate = "gate" in fused
    rows = 2 * n if gate else n
    a, wq, s, z = datagen.wna16_case(m + n + k, m, rows, k, bits, group, zpt)
    z = z if zpt else None
    zp = 1 << (bits - 1)
    rng = np.random.default_rng(5)
    gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float16) if "rms" in fused else None
    bias = rng.standard_normal(n).astype(np.float16) if "bias" in fused else None
    resid = rng.standard_normal((m, n)).astype(np.float16) if "residual" in fused else None
    ta, tw, ts, tz, tg, tb, tr = _t(gpu, a, wq, s, z, gamma, bias, resid)
    out = tr.clone() if fused == "residual-in-place" else None
    y = ops.wna16_gemm_fused(ta, tw, ts, bits=bits, group=group, zp=zp, zero_points=tz, rms_gamma=tg, bias=tb,
                             residual=out if out is not None else tr, act=1 if gate else 0, out=out)
    torch.cuda.synchronize()
    xin = oracle.rmsnorm_f16(a, gamma) if gamma is not None else a
    p = _q_ref(xin, wq, s, bits, group, zp, z)
    if gate:
        _check_gate(y.cpu().numpy(), p, n)
        return
    ref = p
    if bias is not None:
        ref = oracle.add_f16(ref, np.broadcast_to(bias, ref.shape).copy())
    if resid is not None:
        ref = oracle.add_f16(ref, resid)
    _check(y.cpu().numpy(), ref)


@pytest.mark.parametrize("bits,group,zpt", [(4, 32, True), (4, 64, False), (8, 128, True)])
@pytest.mark.parametrize("m", [1, 12, 48, 160])
def test_mlp_block_with_other_block_parameters(gpu, m, bits, group, zpt):
    import torch

    from nnfusion_amd import ops

    h, i = 512, 1408
    x = datagen.normal_f16(7, datagen.S_ACT, (m, h))
    gamma = (1.0 + 0.1 * np.random.default_rng(3).standard_normal(h)).astype(np.float16)
    _, wgu, sgu, zgu = datagen.wna16_case(11, 1, 2 * i, h, bits, group, zpt)
    _, wd, sd, zd = datagen.wna16_case(12, 1, h, i, bits, group, zpt)
    zgu, zd = (zgu, zd) if zpt else (None, None)
    zp = 1 << (bits - 1)
    tx, tg, twgu, tsgu, tzgu, twd, tsd, tzd = _t(gpu, x, gamma, wgu, sgu, zgu, wd, sd, zd)
    out = ops.fused_mlp_wna16(tx, tg, twgu, tsgu, twd, tsd, bits=bits, group=group, zp=zp, zgu=tzgu, zd=tzd)
    inplace = tx.clone()
    ops.fused_mlp_wna16(inplace, tg, twgu, tsgu, twd, tsd, bits=bits, group=group, zp=zp, zgu=tzgu, zd=tzd, out=inplace)
    torch.cuda.synchronize()
    xn = oracle.rmsnorm_f16(x, gamma)
    p = _q_ref(xn, wgu, sgu, bits, group, zp, zgu)
    hh = oracle.silu_mul_f16(p[:, :i].copy(), p[:, i:].copy())
    ref = oracle.add_f16(_q_ref(hh, wd, sd, bits, group, zp, zd), x)
    _check(out.cpu().numpy(), ref)
    assert torch.equal(out, inplace)


def test_plain_parameters_take_the_fused_kernels(gpu):
    """4 bits / groups of 128 / a scalar zero point through the general entry points is the specialised path, bit for bit."""
    import torch

    from nnfusion_amd import ops

    m, h, i = 24, 512, 1408
    x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(2, m, h, i)
    tx, tg, twgu, tsgu, twd, tsd = _t(gpu, x, gamma, wgu, sgu, wd, sd)
    a = ops.fused_mlp_w4a16(tx, tg, twgu, tsgu, twd, tsd)
    b = ops.fused_mlp_wna16(tx, tg, twgu, tsgu, twd, tsd, bits=4, group=128, zp=8)
    c = ops.w4a16_gemm_fused(tx, twgu, tsgu, rms_gamma=tg, act=1)
    d = ops.wna16_gemm_fused(tx, twgu, tsgu, bits=4, group=128, zp=8, rms_gamma=tg, act=1)
    torch.cuda.synchronize()
    assert torch.equal(a, b) and torch.equal(c, d)
