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


def test_onnx_front_door_imports_fuses_and_generates(tmp_path):
    """An ONNX model of the Llama MLP block (SimplifiedLayerNormalization, three MatMulNBits, Sigmoid, Mul, Add) is
    imported, folded into one FusedQuantMLP by the fusion pass and generated as one launcher call; its constants are
    the model's bytes ([gate; up] concatenated by the pass)."""
    from nnfusion_amd import onnx_writer

    m, h, i = 8, 256, 384
    _, gamma, wgu, sgu, wd, sd = datagen.mlp_case(0, m, h, i)
    model = str(tmp_path / "mlp.onnx")
    onnx_writer.write_quant_mlp(model, m, gamma, wgu[:i], sgu[:i], wgu[i:], sgu[i:], wd, sd, 1e-6)
    out = str(tmp_path / "rt") + "/"
    subprocess.run([TOOL, "onnx", out, model], check=True, timeout=60)
    text = open(out + "nnfusion_rt.cpp").read()
    assert text.count("NNF_HIP_CHECK(nnf_") == 1
    assert "nnf_fused_mlp_w4a16_planned(stream, input0, input1," in text and ", 8, 256, 384, 128, 8, " in text
    blobs = {os.path.getsize(out + "Constant/" + c): open(out + "Constant/" + c, "rb").read() for c in os.listdir(out + "Constant")}
    assert blobs[wgu.nbytes] == wgu.tobytes() and blobs[wd.nbytes] == wd.tobytes() and blobs[gamma.nbytes] == gamma.tobytes()
    assert blobs[sgu.nbytes] == sgu.tobytes()
    # a single linear layer becomes one nnf_w4a16_gemm call; unsupported models are refused with the operator's name
    _, wq, s = datagen.w4a16_case(0, 2, 64, 256)
    lin = str(tmp_path / "linear.onnx")
    onnx_writer.write_quant_linear(lin, 2, wq, s)
    out2 = str(tmp_path / "rt2") + "/"
    subprocess.run([TOOL, "onnx", out2, lin], check=True, timeout=60)
    assert "nnf_w4a16_gemm(stream, input0, input1, input2, output0, 2, 64, 256, 128, 8, nullptr, 0)" in open(out2 + "nnfusion_rt.cpp").read()
    # other block parameters: 8 bits, blocks of 64, a zero point per block and fp32 scales go to nnf_wna16_gemm with the
    # zero points as a fourth input; a zero-point tensor that holds one value becomes the scalar of the plain call
    _, wq8, s8, z8 = datagen.wna16_case(0, 2, 64, 256, 8, 64, True)
    onnx_writer.write_quant_linear(lin, 2, wq8, s8.astype(np.float32), bits=8, block=64, zero_points=z8)
    out4 = str(tmp_path / "rt4") + "/"
    subprocess.run([TOOL, "onnx", out4, lin], check=True, timeout=60)
    text = open(out4 + "nnfusion_rt.cpp").read()
    assert "const nnf_quant quant = {8, 64, 0, input3};" in text
    assert "nnf_wna16_gemm(stream, input0, input1, input2, output0, 2, 64, 256, &quant, nullptr, 0)" in text
    blobs = {os.path.getsize(out4 + "Constant/" + c): open(out4 + "Constant/" + c, "rb").read() for c in os.listdir(out4 + "Constant")}
    assert blobs[wq8.nbytes] == wq8.tobytes() and blobs[z8.nbytes] == z8.tobytes() and blobs[s8.nbytes] == s8.tobytes()
    onnx_writer.write_quant_linear(lin, 2, wq, s, zero_points=np.full((64, 1), 0x55, np.uint8))
    out5 = str(tmp_path / "rt5") + "/"
    subprocess.run([TOOL, "onnx", out5, lin], check=True, timeout=60)
    assert "nnf_w4a16_gemm(stream, input0, input1, input2, output0, 2, 64, 256, 128, 5, nullptr, 0)" in open(out5 + "nnfusion_rt.cpp").read()
    _, wq4, s4, z4 = datagen.wna16_case(0, 2, 64, 256, 4, 32, True)
    onnx_writer.write_quant_linear(lin, 2, wq4, s4, bits=4, block=32, zero_points=z4)
    out6 = str(tmp_path / "rt6") + "/"
    subprocess.run([TOOL, "onnx", out6, lin], check=True, timeout=60)
    assert "const nnf_quant quant = {4, 32, 0, input3};" in open(out6 + "nnfusion_rt.cpp").read()
    bad = subprocess.run([TOOL, "onnx", str(tmp_path / "rt3") + "/", os.path.join(ROOT, "tests", "golden", "onnx", "gemm_op.onnx")],
                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert bad.returncode == 1 and "unsupported operator Gemm" in bad.stderr


def _run_generated(name, inputs, out_shape, out_dtype, gpu, n_outputs=1):
    """dlopen nnfusion_amd/generated/<name>, init, kernel_entry(inputs..., outputs...), free.  out_shape: one shape for
    all outputs, or a list of one shape per output."""
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
        shapes = out_shape if isinstance(out_shape, list) else [out_shape] * n_outputs
        n_outputs = len(shapes)
        outs = [torch.empty(sh, dtype=out_dtype, device=gpu) for sh in shapes]
        rt.kernel_entry.argtypes = [ctypes.c_void_p] * (len(dev_in) + n_outputs)
        rt.kernel_entry.restype = ctypes.c_int
        assert rt.kernel_entry(*[t.data_ptr() for t in dev_in], *[o.data_ptr() for o in outs]) == 0
        torch.cuda.synchronize()
        res = outs[0].cpu().numpy() if n_outputs == 1 else [o.cpu().numpy() for o in outs]
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
@pytest.mark.parametrize("name,m,h,i", [("mlp", 16, 256, 384), ("mlp_nodes", 48, 512, 1408), ("mlp_graph", 40, 512, 1024)])
def test_generated_mlp_runtime(gpu, name, m, h, i):
    import torch

    x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(0, m, h, i)
    y = _run_generated(name, [x], (m, h), torch.float16, gpu)
    ref = oracle.fused_mlp_w4a16(x, gamma, wgu, sgu, wd, sd)
    assert np.abs(y.astype(np.float32) - ref.astype(np.float32)).max() <= 1e-2 * _rms(ref)


@pytest.mark.gpu
def test_generated_runtime_of_an_onnx_model(gpu):
    """The runtimes generated at build time from ONNX files (MatMulNBits models written by nnfusion_amd.onnx_writer)."""
    import torch

    import __graft_entry__ as entry

    _, m, h, i = entry.ONNX_EXAMPLES["onnx_mlp"]
    x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(0, m, h, i)
    y = _run_generated("onnx_mlp", [x], (m, h), torch.float16, gpu)
    ref = oracle.fused_mlp_w4a16(x, gamma, wgu, sgu, wd, sd)
    assert np.abs(y.astype(np.float32) - ref.astype(np.float32)).max() <= 1e-2 * _rms(ref)
    _, m, n, k = entry.ONNX_EXAMPLES["onnx_linear"]
    a, wq, s = datagen.w4a16_case(0, m, n, k)
    y = _run_generated("onnx_linear", [a], (m, n), torch.float16, gpu)
    ref = oracle.w4a16_gemm(a, wq, s, f32_out=True)
    assert np.abs(y.astype(np.float32) - ref).max() <= 1e-2 * _rms(ref)
    # 8-bit weights in blocks of 64 with a zero point each (fp32 scales in the file, fp16 on the device)
    _, m, n, k = entry.ONNX_EXAMPLES["onnx_linear_w8"]
    a, wq, s, z = datagen.wna16_case(0, m, n, k, 8, 64, True)
    y = _run_generated("onnx_linear_w8", [a], (m, n), torch.float16, gpu)
    ref = oracle.wna16_gemm(a, wq, s, 8, 64, zero_points=z, f32_out=True)
    assert np.abs(y.astype(np.float32) - ref).max() <= 1e-2 * _rms(ref)
    # 4-bit weights in blocks of 32 with a zero point each, 200 rows: the tile GEMM with the generated code's scratch memory
    _, m, n, k = entry.ONNX_EXAMPLES["onnx_linear_w4z"]
    a, wq, s, z = datagen.wna16_case(0, m, n, k, 4, 32, True)
    y = _run_generated("onnx_linear_w4z", [a], (m, n), torch.float16, gpu)
    ref = oracle.wna16_gemm(a, wq, s, 4, 32, zero_points=z, f32_out=True)
    assert np.abs(y.astype(np.float32) - ref).max() <= 1e-2 * _rms(ref)


@pytest.mark.gpu
def test_generated_qkv_graph_runtime(gpu):
    """RMSNorm feeding three QuantDots: the passes fold the norm in and merge the three into one 3N-row QuantDot
    followed by three Slices; the three results are the column blocks of the wide product."""
    import torch

    m, n, k = 4, 256, 512
    a, wq, s = datagen.w4a16_case(0, m, 3 * n, k)
    gamma = datagen.normal_f16(0, datagen.S_GAMMA, (k,), 1.0, 0.1)
    ys = _run_generated("qkv_graph", [a], (m, n), torch.float16, gpu, n_outputs=3)
    ref = oracle.w4a16_gemm(oracle.rmsnorm_f16(a, gamma, 1e-6), wq, s, f32_out=True)
    src = open(os.path.join(GEN, "qkv_graph", "nnfusion_rt.cpp")).read()
    assert src.count("NNF_HIP_CHECK(nnf_w4a16_gemm") == 1 and src.count("hipMemcpy2DAsync(") == 3
    for i, y in enumerate(ys):
        assert np.abs(y.astype(np.float32) - ref[:, i * n:(i + 1) * n]).max() <= 1e-2 * _rms(ref)


def _gen_src(name):
    return open(os.path.join(GEN, name, "nnfusion_rt.cpp")).read()


@pytest.mark.gpu
def test_generated_runtimes_of_the_other_onnx_forms(gpu):
    """MatMulNBits with a bias; DequantizeLinear + MatMul (the Dequantize -> Dot fold); the MLP block with blocks of 32 and
    zero points (one FusedQuantMLP); and the same block with its gate product as a second result of the graph, which keeps
    RMSNorm-folded products, Sigmoid, two Multiplies and the fused down projection as separate nodes."""
    import torch

    import __graft_entry__ as entry

    tol = 1e-2
    _, m, n, k = entry.ONNX_EXAMPLES["onnx_linear_bias"]
    a, wq, s = datagen.w4a16_case(0, m, n, k)
    bias = datagen.normal_f16(0, datagen.S_BIAS, (n,))
    y = _run_generated("onnx_linear_bias", [a], (m, n), torch.float16, gpu)
    ref = oracle.add_f16(oracle.w4a16_gemm(a, wq, s), np.broadcast_to(bias, (m, n)).copy())
    assert np.abs(y.astype(np.float32) - ref.astype(np.float32)).max() <= tol * _rms(ref)
    assert _gen_src("onnx_linear_bias").count("NNF_HIP_CHECK(nnf_") == 1

    _, m, n, k = entry.ONNX_EXAMPLES["onnx_qdq_u4"]
    a, wq, s, z = datagen.wna16_case(0, m, n, k, 4, 64, True)
    y = _run_generated("onnx_qdq_u4", [a], (m, n), torch.float16, gpu)
    ref = oracle.wna16_gemm(a, wq, s, 4, 64, zero_points=z, f32_out=True)
    assert np.abs(y.astype(np.float32) - ref).max() <= tol * _rms(ref)
    src = _gen_src("onnx_qdq_u4")
    assert src.count("NNF_HIP_CHECK(nnf_") == 1 and "nnf_wna16_gemm(" in src and "nnf_dequantize_f16" not in src

    _, m, n, k = entry.ONNX_EXAMPLES["onnx_qdq_i8"]
    a, wq, s, _ = datagen.wna16_case(0, m, n, k, 8, 128, False)
    y = _run_generated("onnx_qdq_i8", [a], (m, n), torch.float16, gpu)
    ref = oracle.wna16_gemm(a, wq, s, 8, 128, zp=128, f32_out=True)
    assert np.abs(y.astype(np.float32) - ref).max() <= tol * _rms(ref)

    def mlp_reference(m, h, i):
        x, gamma, gate, up, down = entry.mlp_q_case(m, h, i)
        xn = oracle.rmsnorm_f16(x, gamma, 1e-6)
        g = oracle.wna16_gemm(xn, gate[0], gate[1], 4, 32, zero_points=gate[2])
        u = oracle.wna16_gemm(xn, up[0], up[1], 4, 32, zero_points=up[2])
        hh = oracle.silu_mul_f16(g, u)
        return x, g, oracle.add_f16(oracle.wna16_gemm(hh, down[0], down[1], 4, 32, zero_points=down[2]), x)

    _, m, h, i = entry.ONNX_EXAMPLES["onnx_mlp_w4z32"]
    x, _, ref = mlp_reference(m, h, i)
    y = _run_generated("onnx_mlp_w4z32", [x], (m, h), torch.float16, gpu)
    assert np.abs(y.astype(np.float32) - ref.astype(np.float32)).max() <= tol * _rms(ref)
    src = _gen_src("onnx_mlp_w4z32")
    assert src.count("NNF_HIP_CHECK(nnf_") == 1 and "nnf_fused_mlp_wna16(" in src

    _, m, h, i = entry.ONNX_EXAMPLES["onnx_mlp_unfused"]
    x, g_ref, ref = mlp_reference(m, h, i)
    y, g = _run_generated("onnx_mlp_unfused", [x], [(m, h), (m, i)], torch.float16, gpu)
    assert np.abs(g.astype(np.float32) - g_ref.astype(np.float32)).max() <= tol * _rms(g_ref)
    assert np.abs(y.astype(np.float32) - ref.astype(np.float32)).max() <= tol * _rms(ref)
    src = _gen_src("onnx_mlp_unfused")
    # gate and up products with the norm folded in, Sigmoid, Multiply x 2 (one definition: the code generator shares functions
    # with the same signature and body), the down projection with the residual folded in
    assert src.count("NNF_HIP_CHECK(nnf_wna16_gemm_fused(") == 3 and src.count("NNF_HIP_CHECK(nnf_elementwise_f16(") == 2
    assert "NNF_EW_SIGMOID" in src and "NNF_EW_MULTIPLY" in src and "nnf_rms_norm_f16" not in src
