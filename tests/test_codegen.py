"""The HIP code generator end to end.  CPU: the example compiler writes a project that hipcc compiles and
whose shared object exports the generated-runtime C ABI.  GPU: the runtimes generated at build time are
driven the way an external caller drives them (dlopen, rocm_init, kernel_entry with raw device pointers in
para_info.json order, rocm_free) and checked against the oracle."""
import ctypes
import json
import os
import subprocess

import numpy as np
import pytest

import oracle
from nnfusion_amd import datagen

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(ROOT, "nnfusion_amd", "bin", "nnf_compile_example")
GEN = os.path.join(ROOT, "nnfusion_amd", "generated")


def test_generated_project_compiles_and_exports_the_runtime_abi(tmp_path):
    out = str(tmp_path / "rt") + "/"
    inc, lib = os.path.join(ROOT, "include"), os.path.join(ROOT, "nnfusion_amd", "lib")
    subprocess.run([TOOL, "quant_dot", out, "2", "64", "256", inc, lib], check=True, timeout=60)
    for f in ("nnfusion_rt.cpp", "nnfusion_rt.h", "main_test.cpp", "Makefile", "CMakeLists.txt", "para_info.json"):
        assert os.path.exists(out + f), f
    text = open(out + "nnfusion_rt.cpp").read()
    assert "nnf_w4a16_gemm(stream, input0, input1, input2, output0, 2, 64, 256, 128, 8, nullptr, 0)" in text
    for banned in ("cuda_runtime", "cublas", "hipify", "rocm_adapter"):
        assert banned not in text
    subprocess.run(["make", "-C", out, "libnnfusion_rocm_rt.so"], check=True, timeout=300,
                   stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    rt = ctypes.CDLL(out + "libnnfusion_rocm_rt.so")
    for sym in ("kernel_entry", "rocm_init", "rocm_free", "cuda_init", "cuda_free", "get_device_type",
                "get_workspace_size"):
        assert hasattr(rt, sym), sym
    assert rt.get_device_type() == 1  # ROCM_GPU
    info = json.load(open(out + "para_info.json"))
    (in_name, in_info), = info["input"].items()
    assert in_info["shape"] == [2, 256] and in_info["dtype"] == "half"
    (_, out_info), = info["output"].items()
    assert out_info["shape"] == [2, 64]
    consts = sorted(os.listdir(out + "Constant"))
    assert len(consts) == 2 and sum(os.path.getsize(out + "Constant/" + c) for c in consts) == 64 * 128 + 64 * 2 * 2


def _run_generated(name, inputs, out_shape, out_dtype, gpu):
    """dlopen nnfusion_amd/generated/<name>, init, kernel_entry(inputs..., output), free."""
    import torch

    d = os.path.join(GEN, name)
    so = os.path.join(d, "libnnfusion_rocm_rt.so")
    assert os.path.exists(so), f"{so} missing: run build() (python __graft_entry__.py)"
    cwd = os.getcwd()
    os.chdir(d)  # constants are read from ./Constant/
    try:
        rt = ctypes.CDLL(so)
        assert rt.get_device_type() == 1
        rt.rocm_init()
        dev_in = [torch.from_numpy(np.ascontiguousarray(a)).to(gpu) for a in inputs]
        out = torch.empty(out_shape, dtype=out_dtype, device=gpu)
        rt.kernel_entry.argtypes = [ctypes.c_void_p] * (len(dev_in) + 1)
        rt.kernel_entry.restype = ctypes.c_int
        assert rt.kernel_entry(*[t.data_ptr() for t in dev_in], out.data_ptr()) == 0
        torch.cuda.synchronize()
        res = out.cpu().numpy()
        rt.rocm_free()
    finally:
        os.chdir(cwd)
    return res


def _rms(x):
    return float(np.sqrt(np.mean(np.asarray(x, np.float64) ** 2)))


@pytest.mark.gpu
@pytest.mark.parametrize("name,m,n,k", [("quant_dot", 1, 4096, 4096), ("quant_dot_m64", 64, 768, 512)])
def test_generated_quant_dot_runtime(gpu, name, m, n, k):
    import torch

    a, wq, s = datagen.w4a16_case(0, m, n, k)  # the example compiler draws the same constants (seed 0)
    y = _run_generated(name, [a], (m, n), torch.float16, gpu)
    ref = oracle.w4a16_gemm(a, wq, s, f32_out=True)
    assert np.abs(y.astype(np.float32) - ref).max() <= 1e-2 * _rms(ref)


@pytest.mark.gpu
def test_generated_w8a8_runtime(gpu):
    import torch

    m, n, k = 32, 512, 1024
    a, s_tok, w, s_ch = datagen.w8a8_case(0, m, n, k)
    y = _run_generated("w8a8", [a, s_tok], (m, n), torch.float16, gpu)
    assert np.array_equal(y.view(np.uint16), oracle.w8a8_gemm(a, s_tok, w, s_ch).view(np.uint16))


@pytest.mark.gpu
@pytest.mark.parametrize("name,m,h,i", [("mlp", 16, 256, 384), ("mlp_nodes", 48, 512, 1408)])
def test_generated_mlp_runtime(gpu, name, m, h, i):
    import torch

    x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(0, m, h, i)
    y = _run_generated(name, [x], (m, h), torch.float16, gpu)
    ref = oracle.fused_mlp_w4a16(x, gamma, wgu, sgu, wd, sd)
    assert np.abs(y.astype(np.float32) - ref.astype(np.float32)).max() <= 1e-2 * _rms(ref)
