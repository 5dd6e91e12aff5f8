"""The one-launch form of the fp16 x int4 tile GEMM (nnf_plan::sync_flags): the workgroups that share an output tile add
its parts up themselves instead of leaving them to a second launch.

Both forms add the parts in the same order, so the test is bit-for-bit equality with the two-launch form (which the
oracle tests cover), plus the oracle itself, plus the contract of the synchronisation words: all zero again after every
call.  The path taken when a workgroup's wait runs out (its rows handed to the last arriver) is forced from the host
with a negative spin limit; every kernel still ends normally.
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


def _check(y, ref, tol=TOL):
    err = float(np.abs(y.astype(np.float32) - ref.astype(np.float32)).max())
    rms = float(np.sqrt(np.mean(np.asarray(ref, np.float64) ** 2)))
    assert err <= tol * max(rms, 1e-6), (err, rms)


def _ws(gpu, nbytes=96 << 20):
    import torch

    return torch.empty(nbytes, dtype=torch.uint8, device=gpu)


# (tile_rows, k_parts, tile_cols): every tile height and width, tiles shared by 2 .. 5 workgroups, and the library's own
# even split (None), which cuts tiles at arbitrary places
PLANS = [None, (256, 2, 256), (256, 3, 128), (128, 2, 256), (128, 3, 128), (128, 5, 128), (64, 2, 256), (64, 4, 128), (32, 3)]
SHAPES = [(200, 300, 1024), (64, 520, 2048), (130, 128, 1536), (17, 40, 1280), (256, 1024, 4096)]


@pytest.mark.parametrize("spin_limit", [0, -1], ids=["wait", "hand-over"])
@pytest.mark.parametrize("plan", PLANS, ids=lambda p: "auto" if p is None else "rows%d-parts%d" % p[:2] + ("-cols%d" % p[2] if len(p) > 2 else ""))
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_one_launch_equals_two_launches(gpu, m, n, k, plan, spin_limit):
    import torch

    from nnfusion_amd import ops

    print(f"case one-launch M={m} N={n} K={k} plan={plan} spin_limit={spin_limit}", flush=True)
    a, wq, s = datagen.w4a16_case(3, m, n, k)
    ta, tw, ts = _t(gpu, a, wq, s)
    ws = _ws(gpu)
    two = ops.w4a16_gemm_variant(ta, tw, ts, "gemm_mfma", plan=plan, workspace=ws)
    sync = ops.sync_flags(gpu)
    one = ops.w4a16_gemm_variant(ta, tw, ts, "gemm_mfma", plan=plan, workspace=ws, sync=sync, spin_limit=spin_limit)
    torch.cuda.synchronize()
    assert int(sync.count_nonzero()) == 0, "the synchronisation words are zero again after the call"
    assert torch.equal(one, two)
    _check(one.cpu().numpy(), oracle.w4a16_gemm(a, wq, s, f32_out=True))
    # the same buffer again, without clearing it, on a smaller product
    m2 = max(17, m // 2)
    one2 = ops.w4a16_gemm_variant(ta[:m2].contiguous(), tw, ts, "gemm_mfma", plan=plan, workspace=ws, sync=sync, spin_limit=spin_limit)
    two2 = ops.w4a16_gemm_variant(ta[:m2].contiguous(), tw, ts, "gemm_mfma", plan=plan, workspace=ws)
    torch.cuda.synchronize()
    assert int(sync.count_nonzero()) == 0
    assert torch.equal(one2, two2)


@pytest.mark.parametrize("spin_limit", [0, -1], ids=["wait", "hand-over"])
@pytest.mark.parametrize("fused", ["bias+residual", "rms+gate", "rms+bias", "residual-in-place", "rms-whole-tiles"])
def test_one_launch_fused_forms(gpu, fused, spin_limit):
    """With RMSNorm the one-launch form also computes rstd[] inside the GEMM launch (every workgroup a few rows, counted in
    two more synchronisation words; an epilogue whose wait for the count runs out -- forced here with the negative spin
    limit -- adds up the rows it needs itself): the same bits as the pass of its own that the two-launch form runs.
    rms-whole-tiles: no tile is shared (nothing is parked), only rstd[] goes through the synchronisation words."""
    import torch

    from nnfusion_amd import ops

    m, n, k = 150, 384, 2048
    gate = "gate" in fused
    a, wq, s = datagen.w4a16_case(7, m, 2 * n if gate else n, k)
    rng = np.random.default_rng(11)
    gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float16) if "rms" in fused else None
    bias = rng.standard_normal(n).astype(np.float16) if "bias" in fused else None
    resid = rng.standard_normal((m, n)).astype(np.float16) if "residual" in fused else None
    ta, tw, ts, tg, tb, tr = _t(gpu, a, wq, s, gamma, bias, resid)
    kw = dict(rms_gamma=tg, bias=tb, act=1 if gate else 0, variant="gemm_mfma",
              plan=(128, 1 if fused == "rms-whole-tiles" else 3, 256 if gate else 128))
    ws = _ws(gpu)
    if fused == "residual-in-place":
        out_two, out_one = tr.clone(), tr.clone()
        two = ops.w4a16_gemm_fused(ta, tw, ts, residual=out_two, out=out_two, workspace=ws, **kw)
        sync = ops.sync_flags(gpu)
        one = ops.w4a16_gemm_fused(ta, tw, ts, residual=out_one, out=out_one, workspace=ws, sync=sync, spin_limit=spin_limit, **kw)
    else:
        two = ops.w4a16_gemm_fused(ta, tw, ts, residual=tr, workspace=ws, **kw)
        sync = ops.sync_flags(gpu)
        one = ops.w4a16_gemm_fused(ta, tw, ts, residual=tr, workspace=ws, sync=sync, spin_limit=spin_limit, **kw)
    torch.cuda.synchronize()
    assert int(sync.count_nonzero()) == 0
    assert torch.equal(one, two)
    if "rms" in fused and not gate:
        xn = oracle.rmsnorm_f16(a, gamma)
        ref = oracle.w4a16_gemm(xn, wq, s, f32_out=True)
        if bias is not None:
            ref = ref + bias.astype(np.float32)[None, :]
        # the product of the normalised activations; rstd applied to the fp32 sums instead of to fp16 activations
        _check(one.cpu().numpy(), ref, 2e-2)


@pytest.mark.parametrize("m,k", [(300, 1024), (1000, 4096)])
def test_rstd_inside_the_launch_with_more_rows_than_workgroups(gpu, m, k):
    """More activation rows than the launch has workgroups: each adds up the squares of several rows."""
    import torch

    from nnfusion_amd import ops

    n = 512
    a, wq, s = datagen.w4a16_case(4, m, n, k)
    gamma = (1.0 + 0.1 * np.random.default_rng(2).standard_normal(k)).astype(np.float16)
    ta, tw, ts, tg = _t(gpu, a, wq, s, gamma)
    ws = _ws(gpu)
    two = ops.w4a16_gemm_fused(ta, tw, ts, rms_gamma=tg, variant="gemm_mfma", workspace=ws)
    sync = ops.sync_flags(gpu)
    for spin_limit in (0, -1):
        one = ops.w4a16_gemm_fused(ta, tw, ts, rms_gamma=tg, variant="gemm_mfma", workspace=ws, sync=sync, spin_limit=spin_limit)
        torch.cuda.synchronize()
        assert int(sync.count_nonzero()) == 0
        assert torch.equal(one, two)


@pytest.mark.parametrize("spin_limit", [0, -1], ids=["wait", "hand-over"])
@pytest.mark.parametrize("m", [40, 256])
def test_one_launch_mlp_block(gpu, m, spin_limit):
    """The fused MLP with the same synchronisation words for both of its products."""
    import torch

    from nnfusion_amd import ops

    h, i = 1024, 2816
    x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(5, m, h, i)
    tx, tg, twgu, tsgu, twd, tsd = _t(gpu, x, gamma, wgu, sgu, wd, sd)
    two = ops.fused_mlp_w4a16(tx, tg, twgu, tsgu, twd, tsd)
    sync = ops.sync_flags(gpu)
    one = ops.fused_mlp_w4a16(tx, tg, twgu, tsgu, twd, tsd, sync=sync, spin_limit=spin_limit)
    again = ops.fused_mlp_w4a16(tx, tg, twgu, tsgu, twd, tsd, sync=sync, spin_limit=spin_limit)
    torch.cuda.synchronize()
    assert int(sync.count_nonzero()) == 0
    assert torch.equal(one, two) and torch.equal(again, two)


def test_one_launch_full_size_rows(gpu):
    """configs[2] at M = 128 and the MLP block's first product at M = 256, the library's own plans: both forms agree bit for
    bit, twice in a row on the same words."""
    import torch

    from nnfusion_amd import ops

    for (m, n, k) in [(128, 8192, 8192), (256, 4096, 11008)]:
        print(f"case one-launch full size M={m} N={n} K={k}", flush=True)
        a, wq, s = datagen.w4a16_case(1, m, n, k)
        ta, tw, ts = _t(gpu, a, wq, s)
        ws = _ws(gpu)
        two = ops.w4a16_gemm(ta, tw, ts, workspace=ws)
        sync = ops.sync_flags(gpu)
        for _ in range(2):
            one = ops.w4a16_gemm_variant(ta, tw, ts, "auto", workspace=ws, sync=sync)
            torch.cuda.synchronize()
            assert int(sync.count_nonzero()) == 0
            assert torch.equal(one, two)


@pytest.mark.parametrize("fused", ["plain", "bias+residual", "residual-in-place", "rms+bias", "rms"])
@pytest.mark.parametrize("m,n,k", [(16, 4096, 11008), (8, 100, 11008), (3, 520, 16384), (24, 260, 8448), (40, 64, 4352), (12, 33, 13824)])
def test_ranges_of_k_added_up_inside_the_launch(gpu, m, n, k, fused):
    """A few activation rows and K above what one workgroup holds: the row-streaming kernel works on ranges of K; with
    synchronisation words the last workgroup to arrive at a group of columns adds the ranges up, in their order, and runs
    the epilogue -- the same bits as the reduction pass gives (rstd alone included: both round the fp32 product of sum and
    rstd to fp32 before the conversion to fp16), no second launch, the words zero again afterwards.  N not
    a multiple of 16 (a last tile moved back over its neighbour's columns) with the residual in the output buffer: every
    output is written once."""
    import torch

    from nnfusion_amd import ops

    if not ops.w4a16_variant_supported(m, n, k, "gemv_rows"):
        pytest.skip("the row-streaming kernel does not take this shape")
    print(f"case ranges-of-K M={m} N={n} K={k} {fused}", flush=True)
    a, wq, s = datagen.w4a16_case(m + n, m, n, k)
    rng = np.random.default_rng(k)
    gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float16) if "rms" in fused else None
    bias = rng.standard_normal(n).astype(np.float16) if "bias" in fused else None
    resid = rng.standard_normal((m, n)).astype(np.float16) if "residual" in fused else None
    ta, tw, ts, tg, tb, tr = _t(gpu, a, wq, s, gamma, bias, resid)
    ws = _ws(gpu)
    sync = ops.sync_flags(gpu)
    if fused == "plain":
        two = ops.w4a16_gemm_variant(ta, tw, ts, "gemv_rows", workspace=ws)
        one = ops.w4a16_gemm_variant(ta, tw, ts, "gemv_rows", workspace=ws, sync=sync)
        again = ops.w4a16_gemm_variant(ta, tw, ts, "gemv_rows", workspace=ws, sync=sync)
        torch.cuda.synchronize()
        _check(one.cpu().numpy(), oracle.w4a16_gemm(a, wq, s, f32_out=True))
    elif fused == "residual-in-place":
        out_two, out_one, out_again = tr.clone(), tr.clone(), tr.clone()
        two = ops.w4a16_gemm_fused(ta, tw, ts, residual=out_two, out=out_two, variant="gemv_rows", workspace=ws)
        one = ops.w4a16_gemm_fused(ta, tw, ts, residual=out_one, out=out_one, variant="gemv_rows", workspace=ws, sync=sync)
        again = ops.w4a16_gemm_fused(ta, tw, ts, residual=out_again, out=out_again, variant="gemv_rows", workspace=ws, sync=sync)
    else:
        kw = dict(rms_gamma=tg, bias=tb, residual=tr, variant="gemv_rows", workspace=ws)
        two = ops.w4a16_gemm_fused(ta, tw, ts, **kw)
        one = ops.w4a16_gemm_fused(ta, tw, ts, sync=sync, **kw)
        again = ops.w4a16_gemm_fused(ta, tw, ts, sync=sync, **kw)
    torch.cuda.synchronize()
    assert int(sync.count_nonzero()) == 0
    assert torch.equal(one, two) and torch.equal(again, two)


@pytest.mark.parametrize("bits,group,zpt", [(4, 32, True), (4, 64, False), (4, 128, True)])
@pytest.mark.parametrize("m,n,k", [(200, 300, 1024), (64, 520, 2048), (130, 128, 1536), (256, 1024, 4096)])
def test_one_launch_with_other_block_parameters(gpu, m, n, k, bits, group, zpt):
    """nnf_wna16_gemm_planned: the tile GEMM for groups of 32 / 64 / 128 and zero-point tensors in one launch."""
    import torch

    from nnfusion_amd import ops

    a, wq, s, z = datagen.wna16_case(m + k, m, n, k, bits, group, zpt)
    ta, tw, ts, tz = _t(gpu, a, wq, s, z if zpt else None)
    two = ops.wna16_gemm(ta, tw, ts, bits=bits, group=group, zp=8, zero_points=tz)
    sync = ops.sync_flags(gpu)
    for spin_limit in (0, -1):
        one = ops.wna16_gemm(ta, tw, ts, bits=bits, group=group, zp=8, zero_points=tz, sync=sync, spin_limit=spin_limit)
        torch.cuda.synchronize()
        assert int(sync.count_nonzero()) == 0
        assert torch.equal(one, two)
    _check(one.cpu().numpy(), oracle.wna16_gemm(a, wq, s, bits, group, zp=8, zero_points=z if zpt else None).astype(np.float32))


def test_one_launch_random_shapes_and_plans(gpu):
    """Sixty seeded random products -- tile GEMM with any tile shape and split, the row-streaming kernel over ranges of K,
    plain and fused -- four calls each on one set of synchronisation words (the last with the wait forced to run out):
    bit for bit the two-launch result, the words zero after every call."""
    import torch

    from nnfusion_amd import ops

    rng = np.random.default_rng(2024)
    ws = _ws(gpu, 256 << 20)
    sync = ops.sync_flags(gpu)
    done = 0
    for c in range(60):
        if c % 4 == 3:  # a few rows, K above 8192: ranges of K
            m, n, k = int(rng.integers(2, 33)), int(rng.integers(16, 3000)), int(rng.integers(33, 80)) * 256
            plan, variant = None, "gemv_rows"
            if not ops.w4a16_variant_supported(m, n, k, variant):
                continue
        else:
            m, k = int(rng.integers(17, 600)), int(rng.integers(2, 40)) * 128
            n = int(rng.integers(8, 1000)) * 8 if rng.random() < 0.7 else int(rng.integers(17, 3000))
            rows = int(rng.choice([0, 32, 64, 128, 256]))
            cols = int(rng.choice([0, 128, 256])) if rows in (64, 128, 256) else 0
            parts = int(rng.integers(0, 7))
            plan, variant = ((rows, parts, cols) if (rows or parts or cols) else None), "gemm_mfma"
        fused = int(rng.integers(0, 4))  # 0 plain, 1 rms, 2 bias + residual, 3 rms + gate (tile GEMM) / rms (ranges of K)
        gate = fused == 3 and variant == "gemm_mfma"
        print(f"case random {c}: M={m} N={n} K={k} plan={plan} {variant} fused={fused}", flush=True)
        a, wq, s = datagen.w4a16_case(c, m, 2 * n if gate else n, k)
        gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float16) if fused in (1, 3) else None
        bias = rng.standard_normal(n).astype(np.float16) if fused == 2 else None
        resid = rng.standard_normal((m, n)).astype(np.float16) if fused == 2 else None
        ta, tw, ts, tg, tb, tr = _t(gpu, a, wq, s, gamma, bias, resid)
        kw = dict(rms_gamma=tg, bias=tb, residual=tr, act=1 if gate else 0, variant=variant, plan=plan, workspace=ws)
        try:
            two = ops.w4a16_gemm_fused(ta, tw, ts, **kw)
        except ops.NnfError:  # (a plan the shape does not take)
            continue
        for rep in range(4):
            one = ops.w4a16_gemm_fused(ta, tw, ts, sync=sync, spin_limit=-1 if rep == 3 else 0, **kw)
            torch.cuda.synchronize()
            assert int(sync.count_nonzero()) == 0, (c, rep)
            assert torch.equal(one, two), (c, rep, m, n, k, plan, fused)
        done += 1
    assert done >= 40
