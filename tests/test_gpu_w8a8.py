"""W8A8 on the int8 MFMA: the int32 accumulators must be bit-identical to the CPU oracle (pure integer
arithmetic), and the fp16 output identical to fp16((float)acc * s_tok * s_ch) evaluated left to right."""
import numpy as np
import pytest

import oracle
from nnfusion_amd import datagen

pytestmark = pytest.mark.gpu


def _t(gpu, *arrays):
    import torch

    return [torch.from_numpy(np.ascontiguousarray(a)).to(gpu) for a in arrays]


# Kernel families, asked for per call through nnf_w8a8_gemm_variant where the family takes the shape (the library's own
# choice where it does not): "auto"; "skinny": the split-K M <= 16 kernel; "mfma_rows": the row-streaming MFMA kernel
# (2 <= M <= 32, K = 1024 .. 16384 in multiples of 256); otherwise the MFMA tile GEMM with a plan (tile_rows, k_parts):
# tiles of 256 x 256, 256 x 128 (third value: the columns), 128 x 128 or 64 x 256 outputs (0: the library's choice) and the
# number of K ranges (int32 partial sums, added exactly by the reduction pass); "auto-sync": the library's choice given
# synchronisation words (8 .. 32 rows with K from 8192: the row-streaming kernel over two ranges of K in one launch)
@pytest.fixture(params=["auto", "auto-sync", "skinny", "mfma_rows", (0, 0), (256, 1, 256), (256, 2, 256), (256, 1, 128), (256, 3, 128), (256, 0),
                        (128, 1), (128, 3), (64, 1), (64, 2)],
                ids=lambda p: p if isinstance(p, str) else "gemm-rows%d-parts%d" % p[:2] + ("-cols%d" % p[2] if len(p) > 2 else ""))
def path(request):
    return request.param


def _kw(path, m, n, k):
    """Keyword arguments of ops.w8a8_gemm / w8a8_gemm_acc for a fixture value."""
    from nnfusion_amd import ops

    if path == "skinny":
        return {"variant": "gemv_mfma"} if ops.w8a8_variant_supported(m, n, k, "gemv_mfma") else {}
    if path == "mfma_rows":
        return {"variant": "gemv_rows"} if m > 1 and ops.w8a8_variant_supported(m, n, k, "gemv_rows") else {}
    if path == "auto":
        return {}
    if path == "auto-sync":
        import torch

        return {"sync": ops.sync_flags(torch.device("cuda:0"))}
    return {"variant": "gemm_mfma", "plan": path}


def _words_left_zero(kw):
    return "sync" not in kw or int(kw["sync"].count_nonzero()) == 0


def _big_ws(gpu):
    import torch

    return torch.empty(64 << 20, dtype=torch.uint8, device=gpu)


@pytest.mark.parametrize("m,n,k", [
    (1, 64, 128), (1, 1000, 1024), (3, 17, 256), (16, 512, 8192), (32, 300, 512), (100, 257, 384),
    (256, 256, 128), (512, 1024, 2048), (1, 8192, 8192), (32, 4096, 4096),
    # M <= 16 with chunk counts that leave wavefronts partly idle, two passes over K per tile, many tiles
    (5, 200, 2176), (2, 100, 11008), (7, 48, 16384), (9, 1000, 8320), (1, 33000, 1024), (13, 8200, 4096),
    # ... and with K so short that the workgroup has fewer threads than a tile has outputs (two wavefronts, 9 .. 16 rows)
    (14, 4128, 128), (9, 100, 128), (16, 300, 128), (13, 64, 128), (8, 520, 128), (12, 1000, 128),
    # one activation row: rows shared by 1..8 wavefronts, ragged last K segment, fewer rows than wavefronts
    (1, 300, 4096), (1, 4096, 11008), (1, 100, 16384), (1, 50, 2048), (1, 513, 5248), (1, 2000, 24576), (1, 40, 1152),
    # 2 .. 32 rows through the row-streaming MFMA kernel: every K it takes, one and two blocks of 16 rows, ragged N,
    # a single tile, more tiles than CUs
    (2, 512, 2048), (16, 4111, 4096), (17, 1000, 6144), (32, 8192, 8192), (31, 16, 8192), (24, 12288, 4096),
    (8, 40000, 2048), (20, 77, 4096),
    # K that does not fill the last 2-KiB step, K above 8192
    (16, 4111, 11008), (5, 100, 1024), (9, 520, 2560), (32, 300, 7168), (24, 1000, 3584), (12, 2000, 14336), (16, 64, 16384),
    (17, 250, 5376), (32, 4111, 11008), (20, 300, 12288), (24, 100, 9216),
    # two ranges of K given synchronisation words: one to four tiles per workgroup, a last tile moved back, K = 16384
    (8, 4096, 8192), (32, 4111, 8192), (13, 6000, 16384), (24, 8192, 9216),
])
def test_accumulators_bit_exact(gpu, path, m, n, k):
    import torch

    from nnfusion_amd import ops

    print(f"case M={m} N={n} K={k} path={path}", flush=True)
    a, s_tok, w, s_ch = datagen.w8a8_case(0, m, n, k)
    ta, tw, tst, tsc = _t(gpu, a, w, s_tok, s_ch)
    ws = _big_ws(gpu)
    kw = _kw(path, m, n, k)
    acc = ops.w8a8_gemm_acc(ta, tw, workspace=ws, **kw).cpu().numpy()
    y = ops.w8a8_gemm(ta, tst, tw, tsc, workspace=ws, **kw).cpu().numpy()
    torch.cuda.synchronize()
    ref = oracle.w8a8_acc(a, w)
    assert np.array_equal(acc, ref)
    # the epilogue is a closed form of exact inputs: bit-identical fp16
    assert np.array_equal(y.view(np.uint16), oracle.w8a8_epilogue(ref, s_tok, s_ch).view(np.uint16))
    assert _words_left_zero(kw)


def test_extreme_values_do_not_overflow(gpu, path):
    """All operands at -127 / +127 with K = 8192: |acc| = 8192 * 127^2 = 132 128 768 < 2^31."""
    import torch

    from nnfusion_amd import ops

    m, n, k = 4, 48, 8192
    a = np.full((m, k), 127, np.int8)
    a[1] = -127
    w = np.full((n, k), 127, np.int8)
    w[::2] = -127
    ta, tw = _t(gpu, a, w)
    kw = _kw(path, m, n, k)
    acc = ops.w8a8_gemm_acc(ta, tw, workspace=_big_ws(gpu), **kw).cpu().numpy()
    torch.cuda.synchronize()
    assert np.array_equal(acc, oracle.w8a8_acc(a, w))
    assert _words_left_zero(kw)
    assert abs(int(acc[0, 1])) == 8192 * 127 * 127


@pytest.mark.parametrize("m", [512, 4096])
def test_full_size_sampled(gpu, m):
    """configs[3] at N = K = 8192: sampled output columns against the oracle bit for bit, and the
    checksum identity  sum_n acc[m, n] == A[m, :] . (sum_n W[n, :])  over the whole output in int64."""
    import torch

    from nnfusion_amd import ops

    n = k = 8192
    print(f"case M={m}", flush=True)
    a, s_tok, w, s_ch = datagen.w8a8_case(0, m, n, k)
    ta, tw = _t(gpu, a, w)
    acc = ops.w8a8_gemm_acc(ta, tw).cpu().numpy()
    torch.cuda.synchronize()
    cols = np.sort(np.random.default_rng(1).choice(n, 128, replace=False))
    assert np.array_equal(acc[:, cols], oracle.w8a8_acc(a, w[cols]))
    wsum = w.astype(np.int64).sum(axis=0)
    assert np.array_equal(acc.astype(np.int64).sum(axis=1), a.astype(np.int64) @ wsum)
