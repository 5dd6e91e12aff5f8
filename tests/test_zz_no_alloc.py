"""nnf_w4a16_gemm_static_scratch (the entry point that allocates nothing and takes no workspace) against
nnf_w4a16_gemm on the same inputs: same kernels, so the fp16 results must be bit-identical.

Two calls in a row on shapes whose plan writes partial sums to scratch memory, the second one smaller: the
library's static buffer keeps the first call's contents, and nothing of them may leak into the second result.
"""
import numpy as np
import pytest

from nnfusion_amd import datagen

pytestmark = pytest.mark.gpu

STATIC_SCRATCH_BYTES = 32 << 20


def _static(gpu, ta, tw, ts, m, n, k):
    import torch

    from nnfusion_amd import _lib, ops

    lib = _lib.kernels()
    y = torch.full((m, n), float("nan"), dtype=torch.float16, device=gpu)
    st = lib.nnf_w4a16_gemm_static_scratch(torch.cuda.current_stream().cuda_stream, ta.data_ptr(), tw.data_ptr(),
                                           ts.data_ptr(), y.data_ptr(), m, n, k, 128, 8)
    if st != 0:
        raise ops.NnfError(st, "nnf_w4a16_gemm_static_scratch")
    return y


def test_static_scratch_matches_workspace_entry_point_twice(gpu):
    import torch

    from nnfusion_amd import _lib, ops

    lib = _lib.kernels()
    # (M, N, K): tile GEMM over 4 K ranges (16 MiB of partial sums), then smaller: 8 K ranges (4 MiB),
    # then the row-streaming MFMA kernel over 3 ranges of K (M = 16)
    for (m, n, k) in [(128, 8192, 8192), (64, 2048, 4096), (16, 260, 11008)]:
        print(f"case M={m} N={n} K={k}", flush=True)
        need = lib.nnf_w4a16_gemm_workspace_bytes(m, n, k, 128)
        assert 0 < need <= STATIC_SCRATCH_BYTES, need  # the shape does use scratch memory
        a, wq, s = datagen.w4a16_case(5, m, n, k)
        ta, tw, ts = [torch.from_numpy(x).to(gpu) for x in (a, wq, s)]
        y_ws = ops.w4a16_gemm(ta, tw, ts)
        y_st = _static(gpu, ta, tw, ts, m, n, k)
        torch.cuda.synchronize()
        assert np.array_equal(y_st.cpu().numpy().view(np.uint16), y_ws.cpu().numpy().view(np.uint16)), (m, n, k)


def test_static_scratch_rejects_shapes_beyond_its_buffer(gpu):
    import torch

    from nnfusion_amd import _lib

    lib = _lib.kernels()
    m, n, k = 384, 22016, 4096
    assert lib.nnf_w4a16_gemm_workspace_bytes(m, n, k, 128) > STATIC_SCRATCH_BYTES
    t = torch.zeros(256, dtype=torch.uint8, device=gpu)  # never touched: the call is refused on its shape
    st = lib.nnf_w4a16_gemm_static_scratch(torch.cuda.current_stream().cuda_stream, t.data_ptr(), t.data_ptr(),
                                           t.data_ptr(), t.data_ptr(), m, n, k, 128, 8)
    assert st == -5
    assert b"static" in lib.nnf_status_string(st)
