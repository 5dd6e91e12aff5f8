"""Fused Llama-style MLP block (RMSNorm -> gate|up -> SiLU*mul -> down -> +residual) against the oracle's
unfused graph with fp16 tensors between the nodes.  Tolerance: 1e-2 * RMS(out) on the block output."""
import numpy as np
import pytest

import oracle
from nnfusion_amd import datagen

pytestmark = pytest.mark.gpu


def _t(gpu, *arrays):
    import torch

    return [torch.from_numpy(np.ascontiguousarray(a)).to(gpu) for a in arrays]


def _rms(x):
    return float(np.sqrt(np.mean(np.asarray(x, np.float64) ** 2)))


# the last four: the decode route (GEMV kernels with element-wise epilogues; M = 1, a few rows, two blocks of 16 rows,
# a down projection over ranges of K)
@pytest.mark.parametrize("m,h,i", [(64, 256, 384), (256, 512, 1408), (37, 1024, 2816), (1, 1024, 2816), (8, 2048, 5632),
                                   (24, 1024, 2816), (16, 1024, 8704)])
def test_mlp_matches_unfused_oracle(gpu, m, h, i):
    import torch

    from nnfusion_amd import ops

    x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(0, m, h, i)
    out = ops.fused_mlp_w4a16(*_t(gpu, x, gamma, wgu, sgu, wd, sd)).cpu().numpy()
    torch.cuda.synchronize()
    ref = oracle.fused_mlp_w4a16(x, gamma, wgu, sgu, wd, sd)
    err = float(np.abs(out.astype(np.float32) - ref.astype(np.float32)).max())
    assert err <= 1e-2 * _rms(ref), (err, _rms(ref))


def test_mlp_full_size_rows(gpu):
    """configs[4]: M = 256, 4096 -> 11008 -> 4096.  The oracle runs the first 8 token rows (rows are
    independent); the other rows are covered by duplicated rows, which must give the same outputs up to the
    rounding of a different summation order (the rows sit in different tiles, whose K ranges are cut at different
    places by the even split of the work over the CUs; run to run the result is bit-identical: see below)."""
    import torch

    from nnfusion_amd import ops

    m, h, i = 256, 4096, 11008
    x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(0, m, h, i)
    x[128:136] = x[0:8]  # duplicated tokens must give duplicated outputs (different tile rows)
    out = ops.fused_mlp_w4a16(*_t(gpu, x, gamma, wgu, sgu, wd, sd)).cpu().numpy()
    torch.cuda.synchronize()
    ref = oracle.fused_mlp_w4a16(x[:8].copy(), gamma, wgu, sgu, wd, sd)
    err = float(np.abs(out[:8].astype(np.float32) - ref.astype(np.float32)).max())
    assert err <= 1e-2 * _rms(ref), (err, _rms(ref))
    dup = float(np.abs(out[128:136].astype(np.float32) - out[0:8].astype(np.float32)).max())
    assert dup <= 2e-3 * _rms(ref), (dup, _rms(ref))
    again = ops.fused_mlp_w4a16(*_t(gpu, x, gamma, wgu, sgu, wd, sd)).cpu().numpy()
    assert np.array_equal(again, out)


@pytest.mark.parametrize("m,h,i", [(1, 1024, 2816), (4, 1024, 11008), (16, 2048, 5632), (24, 1024, 2816),
                                   (16, 1024, 8704), (64, 512, 1408)])
def test_mlp_output_may_be_the_input_buffer(gpu, m, h, i):
    """out == x: the residual of the down projection is then the output buffer itself (the decode kernels add it in
    place at their flush; the MFMA GEMV kernel goes through scratch memory; the tile GEMM reads each element before it
    writes it).  Same results as with a separate output."""
    import torch

    from nnfusion_amd import ops

    tens = _t(gpu, *datagen.mlp_case(2, m, h, i))
    want = ops.fused_mlp_w4a16(*tens)
    x = tens[0].clone()
    got = ops.fused_mlp_w4a16(x, *tens[1:], out=x)
    torch.cuda.synchronize()
    assert got.data_ptr() == x.data_ptr()
    assert torch.equal(got, want)


def test_mlp_workspace_contract(gpu):
    import torch

    from nnfusion_amd import _lib, ops

    m, h, i = 32, 256, 384
    tens = _t(gpu, *datagen.mlp_case(1, m, h, i))
    need = _lib.kernels().nnf_fused_mlp_w4a16_workspace_bytes(m, h, i, 128)
    assert need >= m * i * 2
    # the query is an upper bound over the kernels the library may pick; a call checks what its own launches write:
    # always the block's h tensor, which alone is M x I fp16
    small = torch.empty(m * i * 2 - 256, dtype=torch.uint8, device=gpu)
    with pytest.raises(ops.NnfError) as e:
        ops.fused_mlp_w4a16(*tens, workspace=small)
    assert e.value.status == -3
