"""Writes small ONNX models of the quantized path (com.microsoft::MatMulNBits) without the
`onnx` package: a minimal encoder of the protobuf wire format for the messages of onnx.proto3 that such a model
needs.  The layouts are those of the operator: B = uint8 [N, K/128, 64] with the even k in the low nibble, scales
[N * K/128], which is byte for byte the `Wq [N, K/2]` / `scales [N, K/128]` layout of include/nnf_hip_kernels.h.
"""
import struct

import numpy as np

FLOAT, UINT8, FLOAT16 = 1, 2, 10
ATTR_FLOAT, ATTR_INT = 1, 2


def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _key(field, wire):
    return _varint((field << 3) | wire)


def _int(field, v):
    return _key(field, 0) + _varint(v)


def _bytes(field, b):
    return _key(field, 2) + _varint(len(b)) + bytes(b)


def _str(field, s):
    return _bytes(field, s.encode())


def _tensor(name, array, data_type, dims=None):
    """TensorProto with raw_data (little endian, the tensor's own element type)."""
    a = np.ascontiguousarray(array)
    msg = b"".join(_int(1, d) for d in (a.shape if dims is None else dims))
    msg += _int(2, data_type) + _str(8, name) + _bytes(9, a.tobytes())
    return msg


def _value_info(name, elem_type, dims):
    shape = b"".join(_bytes(1, _int(1, d)) for d in dims)          # TensorShapeProto.dim[].dim_value
    tensor_type = _int(1, elem_type) + _bytes(2, shape)             # TypeProto.Tensor
    return _str(1, name) + _bytes(2, _bytes(1, tensor_type))       # ValueInfoProto{name, type{tensor_type}}


def _attr_int(name, v):
    return _str(1, name) + _int(3, v) + _int(20, ATTR_INT)


def _attr_float(name, v):
    return _str(1, name) + _key(2, 5) + struct.pack("<f", v) + _int(20, ATTR_FLOAT)


def _node(op_type, inputs, outputs, name, attrs=(), domain=""):
    msg = b"".join(_str(1, i) for i in inputs) + b"".join(_str(2, o) for o in outputs)
    msg += _str(3, name) + _str(4, op_type) + b"".join(_bytes(5, a) for a in attrs)
    if domain:
        msg += _str(7, domain)
    return msg


def _matmul_nbits(name, a, w_name, s_name, out, n, k, bits=4, block=128, z_name=None):
    return _node("MatMulNBits", [a, w_name, s_name] + ([z_name] if z_name else []), [out], name,
                 [_attr_int("K", k), _attr_int("N", n), _attr_int("bits", bits), _attr_int("block_size", block)],
                 domain="com.microsoft")


def _model(graph_name, nodes, initializers, inputs, outputs):
    graph = b"".join(_bytes(1, n) for n in nodes) + _str(2, graph_name)
    graph += b"".join(_bytes(5, t) for t in initializers)
    graph += b"".join(_bytes(11, v) for v in inputs) + b"".join(_bytes(12, v) for v in outputs)
    model = _int(1, 8) + _str(2, "nnfusion_amd.onnx_writer") + _bytes(7, graph)
    model += _bytes(8, _str(1, "") + _int(2, 17))               # default domain, opset 17
    model += _bytes(8, _str(1, "com.microsoft") + _int(2, 1))
    return model


def _weights(prefix, wq, scales):
    n, half_k = wq.shape
    k = half_k * 2
    assert wq.dtype == np.uint8 and scales.dtype == np.float16 and scales.shape == (n, k // 128)
    return [_tensor(prefix + "_B", wq, UINT8, dims=(n, k // 128, 64)),
            _tensor(prefix + "_scales", scales.reshape(-1), FLOAT16)], n, k


def write_quant_linear(path, m, wq, scales, bits=4, block=128, zero_points=None):
    """y [m, N] = MatMulNBits(x [m, K], B, scales[, zero_points]); scales fp16 or fp32 [N, K/block], zero_points u8
    [N, ceil(K/block*bits/8)] (4-bit ones two per byte, even block in the low nibble)."""
    if (bits, block) == (4, 128) and zero_points is None and scales.dtype == np.float16:
        inits, n, k = _weights("linear", wq, scales)
    else:
        n, k = wq.shape[0], wq.shape[1] * 8 // bits
        assert wq.dtype == np.uint8 and scales.shape == (n, k // block) and scales.dtype in (np.float16, np.float32)
        inits = [_tensor("linear_B", wq, UINT8, dims=(n, k // block, block * bits // 8)),
                 _tensor("linear_scales", scales.reshape(-1), FLOAT16 if scales.dtype == np.float16 else FLOAT)]
        if zero_points is not None:
            assert zero_points.dtype == np.uint8 and zero_points.shape == (n, (k // block * bits + 7) // 8)
            inits.append(_tensor("linear_zp", zero_points.reshape(-1), UINT8))
    nodes = [_matmul_nbits("linear", "x", "linear_B", "linear_scales", "y", n, k, bits, block,
                           "linear_zp" if zero_points is not None else None)]
    data = _model("quant_linear", nodes, inits, [_value_info("x", FLOAT16, (m, k))], [_value_info("y", FLOAT16, (m, n))])
    with open(path, "wb") as f:
        f.write(data)


def write_quant_mlp(path, m, gamma, w_gate, s_gate, w_up, s_up, w_down, s_down, eps=1e-6):
    """The Llama MLP block: out = x + down(silu(gate(norm(x))) * up(norm(x))), norm = SimplifiedLayerNormalization."""
    inits = [_tensor("gamma", gamma, FLOAT16)]
    ig, i_dim, h_dim = _weights("gate", w_gate, s_gate)
    iu, _, _ = _weights("up", w_up, s_up)
    idn, h2, i2 = _weights("down", w_down, s_down)
    assert (h2, i2) == (h_dim, i_dim) and gamma.shape == (h_dim,) and gamma.dtype == np.float16
    inits += ig + iu + idn
    nodes = [
        _node("SimplifiedLayerNormalization", ["x", "gamma"], ["n"], "norm", [_attr_int("axis", -1), _attr_float("epsilon", eps)]),
        _matmul_nbits("gate", "n", "gate_B", "gate_scales", "g", i_dim, h_dim),
        _matmul_nbits("up", "n", "up_B", "up_scales", "u", i_dim, h_dim),
        _node("Sigmoid", ["g"], ["sg"], "sigmoid"),
        _node("Mul", ["g", "sg"], ["act"], "silu"),
        _node("Mul", ["act", "u"], ["h"], "gated"),
        _matmul_nbits("down", "h", "down_B", "down_scales", "d", h_dim, i_dim),
        _node("Add", ["x", "d"], ["out"], "residual"),
    ]
    data = _model("quant_mlp", nodes, inits, [_value_info("x", FLOAT16, (m, h_dim))], [_value_info("out", FLOAT16, (m, h_dim))])
    with open(path, "wb") as f:
        f.write(data)
