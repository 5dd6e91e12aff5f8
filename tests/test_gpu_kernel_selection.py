"""Profiling-based kernel selection (the reference's ProfilingBasedKernelSelector,
src/nnfusion/engine/pass/graph/kernel_selection.cpp:21-137) on QuantDot nodes: every registered emitter that
accepts the node runs through the single-kernel harness (built ahead of time by __graft_entry__.build()) and the
fastest is kept.  The candidates ran on the same inputs: their results have to agree."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402


def _select(name):
    cmd = entry.kernel_selection_command("run", name)
    assert os.path.exists(cmd[0]), "run __graft_entry__.build() first"
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    return json.loads(proc.stdout.strip().splitlines()[-1])


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(entry.KERNEL_SELECTION_SHAPES))
def test_profiling_selector_times_every_candidate_and_keeps_the_fastest(gpu, name):
    m, n, k = entry.KERNEL_SELECTION_SHAPES[name]
    res = _select(name)
    kinds = {c["kernel"] for c in res["candidates"]}
    expected = {"rocm", "rocm_gemm_mfma"}
    if m <= 16:
        expected |= {"rocm_gemv_mfma", "rocm_gemv_valu"}
    if m <= 16:  # the row-streaming kernels: one row, or 2 .. 16 rows at K = 1024, 1280 .. 8192
        expected.add("rocm_gemv_rows")
    assert kinds == expected
    assert all(c["ms"] > 0 for c in res["candidates"]), res
    assert res["ran"] == len(expected)
    times = {c["kernel"]: c["ms"] for c in res["candidates"]}
    # (two candidates may run the same kernel and tie at the printed precision)
    assert times[res["best"]] == min(times.values())
    # same inputs, same product: fp16 results within a few ulps of each other (different summation orders)
    assert res["max_abs_diff"] <= 2e-2 * max(res["max_abs_ref"], 1e-3), res
    if m == 1:
        # a single row: the streaming GEMV kernels, never the MFMA tile GEMM
        assert res["best"] in ("rocm", "rocm_gemv_rows", "rocm_gemv_mfma"), res
        assert times["rocm_gemm_mfma"] > times[res["best"]]


@pytest.mark.gpu
def test_code_generation_with_kernel_selection_emits_the_fastest_candidate(gpu, tmp_path):
    """The compile flow with -fkernel_selection semantics: device dispatch, profiling of every QuantDot candidate (the
    harness objects were built by build()), then the default selector keeps the profiled winner and the code
    generator emits that kernel's call."""
    out = str(tmp_path / "rt") + "/"
    cmd = entry.compile_with_kernel_selection_command(out, False)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    text = open(out + "nnfusion_rt.cpp").read()
    calls = [l.strip() for l in text.splitlines() if "NNF_HIP_CHECK(nnf_" in l]
    assert len(calls) == 1, calls
    # one activation row: a streaming GEMV kernel wins (the automatic emitter resolves to the same kernel as gemv_rows)
    assert ("nnf_w4a16_gemm(stream" in calls[0] or "NNF_W4A16_GEMV_ROWS" in calls[0] or "NNF_W4A16_GEMV_MFMA" in calls[0]), calls
    timed = [l for l in proc.stderr.splitlines() + proc.stdout.splitlines() if "time cost(ms)" in l]
    assert len(timed) == 5, proc.stderr[-2000:]
