"""Writes small ONNX models of the quantized path (com.microsoft::MatMulNBits) without the
`onnx` package: a minimal encoder of the protobuf wire format for the messages of onnx.proto3 that such a model
needs.  The layouts are those of the operator: B = uint8 [N, K/128, 64] with the even k in the low nibble, scales
[N * K/128], which is byte for byte the `Wq [N, K/2]` / `scales [N, K/128]` layout of include/nnf_hip_kernels.h.
"""
import struct

import numpy as np

FLOAT, UINT8, INT8, FLOAT16, UINT4, INT4 = 1, 2, 3, 10, 21, 22
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


def _matmul_nbits(name, a, w_name, s_name, out, n, k, bits=4, block=128, z_name=None, bias_name=None):
    ins = [a, w_name, s_name]
    if z_name or bias_name:
        ins += [z_name or "", "" if bias_name else None, bias_name]  # inputs 3 zero_points, 4 g_idx (absent), 5 bias
    return _node("MatMulNBits", [i for i in ins if i is not None], [out], name,
                 [_attr_int("K", k), _attr_int("N", n), _attr_int("bits", bits), _attr_int("block_size", block)],
                 domain="com.microsoft")


def _model(graph_name, nodes, initializers, inputs, outputs, opset=17):
    graph = b"".join(_bytes(1, n) for n in nodes) + _str(2, graph_name)
    graph += b"".join(_bytes(5, t) for t in initializers)
    graph += b"".join(_bytes(11, v) for v in inputs) + b"".join(_bytes(12, v) for v in outputs)
    model = _int(1, 8) + _str(2, "nnfusion_amd.onnx_writer") + _bytes(7, graph)
    model += _bytes(8, _str(1, "") + _int(2, opset))            # default domain
    model += _bytes(8, _str(1, "com.microsoft") + _int(2, 1))
    return model


def _weights(prefix, wq, scales):
    n, half_k = wq.shape
    k = half_k * 2
    assert wq.dtype == np.uint8 and scales.dtype == np.float16 and scales.shape == (n, k // 128)
    return [_tensor(prefix + "_B", wq, UINT8, dims=(n, k // 128, 64)),
            _tensor(prefix + "_scales", scales.reshape(-1), FLOAT16)], n, k


def _weights_q(prefix, wq, scales, bits, block, zero_points):
    """Initializers of one MatMulNBits with any block parameters; returns (initializers, N, K, zero-point name or None)."""
    n, k = wq.shape[0], wq.shape[1] * 8 // bits
    assert wq.dtype == np.uint8 and scales.shape == (n, k // block) and scales.dtype in (np.float16, np.float32)
    inits = [_tensor(prefix + "_B", wq, UINT8, dims=(n, k // block, block * bits // 8)),
             _tensor(prefix + "_scales", scales.reshape(-1), FLOAT16 if scales.dtype == np.float16 else FLOAT)]
    if zero_points is not None:
        assert zero_points.dtype == np.uint8 and zero_points.shape == (n, (k // block * bits + 7) // 8)
        inits.append(_tensor(prefix + "_zp", zero_points.reshape(-1), UINT8))
    return inits, n, k, (prefix + "_zp" if zero_points is not None else None)


def write_quant_linear(path, m, wq, scales, bits=4, block=128, zero_points=None, bias=None):
    """y [m, N] = MatMulNBits(x [m, K], B, scales[, zero_points][, bias]); scales fp16 or fp32 [N, K/block], zero_points u8
    [N, ceil(K/block*bits/8)] (4-bit ones two per byte, even block in the low nibble), bias fp16 or fp32 [N]."""
    if (bits, block) == (4, 128) and zero_points is None and scales.dtype == np.float16:
        inits, n, k = _weights("linear", wq, scales)
    else:
        inits, n, k, _ = _weights_q("linear", wq, scales, bits, block, zero_points)
    if bias is not None:
        assert bias.shape == (n,) and bias.dtype in (np.float16, np.float32)
        inits.append(_tensor("linear_bias", bias, FLOAT16 if bias.dtype == np.float16 else FLOAT))
    nodes = [_matmul_nbits("linear", "x", "linear_B", "linear_scales", "y", n, k, bits, block,
                           "linear_zp" if zero_points is not None else None, "linear_bias" if bias is not None else None)]
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


def write_quant_mlp_q(path, m, gamma, gate, up, down, bits, block, eps=1e-6, extra_outputs=()):
    """The same block with any block parameters: gate / up / down = (wq u8 [N, K*bits/8], scales [N, K/block], zero points or
    None).  extra_outputs: names among n (the normalised input), g (gate product), u, act, h, d to return as well -- a value
    with a second consumer cannot be folded away, so the nodes around it stay nodes."""
    inits = [_tensor("gamma", gamma, FLOAT16)]
    ig, i_dim, h_dim, zg = _weights_q("gate", gate[0], gate[1], bits, block, gate[2])
    iu, _, _, zu = _weights_q("up", up[0], up[1], bits, block, up[2])
    idn, h2, i2, zd = _weights_q("down", down[0], down[1], bits, block, down[2])
    assert (h2, i2) == (h_dim, i_dim) and gamma.shape == (h_dim,) and gamma.dtype == np.float16
    inits += ig + iu + idn
    nodes = [
        _node("SimplifiedLayerNormalization", ["x", "gamma"], ["n"], "norm", [_attr_int("axis", -1), _attr_float("epsilon", eps)]),
        _matmul_nbits("gate", "n", "gate_B", "gate_scales", "g", i_dim, h_dim, bits, block, zg),
        _matmul_nbits("up", "n", "up_B", "up_scales", "u", i_dim, h_dim, bits, block, zu),
        _node("Sigmoid", ["g"], ["sg"], "sigmoid"),
        _node("Mul", ["g", "sg"], ["act"], "silu"),
        _node("Mul", ["act", "u"], ["h"], "gated"),
        _matmul_nbits("down", "h", "down_B", "down_scales", "d", h_dim, i_dim, bits, block, zd),
        _node("Add", ["x", "d"], ["out"], "residual"),
    ]
    widths = {"n": h_dim, "g": i_dim, "u": i_dim, "act": i_dim, "h": i_dim, "d": h_dim}
    outputs = [_value_info("out", FLOAT16, (m, h_dim))] + [_value_info(o, FLOAT16, (m, widths[o])) for o in extra_outputs]
    data = _model("quant_mlp", nodes, inits, [_value_info("x", FLOAT16, (m, h_dim))], outputs)
    with open(path, "wb") as f:
        f.write(data)


def _pack4(values):
    """Flat array of 4-bit values -> bytes, the first of each pair in the low nibble (ONNX's packing of (u)int4 tensors)."""
    v = np.asarray(values, np.uint8).reshape(-1) & 0xF
    if v.size & 1:
        v = np.concatenate([v, np.zeros(1, np.uint8)])
    return (v[0::2] | (v[1::2] << 4)).astype(np.uint8)


def write_qdq_linear(path, m, wq, scales, bits=4, block=128, zero_points=None, signed=False):
    """y [m, N] = MatMul(x [m, K], DequantizeLinear(W [K, N], scale [K/block, N][, zero point], axis = 0, block_size = block)):
    the QDQ form of a weight-quantized linear layer (opset 21).  Arguments in the layout of the kernels -- wq u8
    [N, K*bits/8], scales [N, K/block], zero_points u8 [N, ceil(K/block*bits/8)] or None (= 2^(bits-1) everywhere) -- and
    converted here to the operator's: the weight matrix transposed, 4-bit values two per byte in row-major order of
    [K, N].  signed: stored as int4 / int8 (every value minus 2^(bits-1)); a zero point of 2^(bits-1) everywhere is then
    the operator's default of 0 and no zero-point tensor is written."""
    n, k = wq.shape[0], wq.shape[1] * 8 // bits
    g = k // block
    half = 1 << (bits - 1)
    if bits == 4:
        q = np.stack([wq & 0xF, wq >> 4], axis=-1).reshape(n, k).astype(np.int32)
    else:
        q = wq.astype(np.int32)
    q_kn = np.ascontiguousarray(q.T)  # [K, N]
    z_gn = None
    if zero_points is not None:
        if bits == 4:
            z = np.stack([zero_points & 0xF, zero_points >> 4], axis=-1).reshape(n, -1)[:, :g].astype(np.int32)
        else:
            z = zero_points.astype(np.int32)
        z_gn = np.ascontiguousarray(z.T)
    elif not signed:
        z_gn = np.full((g, n), half, np.int32)  # unsigned storage: the zero point has to be spelled out
    if signed:
        q_kn = q_kn - half
        z_gn = None if z_gn is None else z_gn - half
    dt = {(4, False): UINT4, (4, True): INT4, (8, False): UINT8, (8, True): INT8}[(bits, signed)]

    def raw(values):
        return _pack4(values) if bits == 4 else np.asarray(values, np.int8 if signed else np.uint8).reshape(-1).view(np.uint8)

    inits = [_tensor("W_q", raw(q_kn), dt, dims=(k, n)),
             _tensor("W_scale", np.ascontiguousarray(scales.T), FLOAT16 if scales.dtype == np.float16 else FLOAT)]
    dq_inputs = ["W_q", "W_scale"]
    if z_gn is not None:
        inits.append(_tensor("W_zp", raw(z_gn), dt, dims=(g, n)))
        dq_inputs.append("W_zp")
    nodes = [_node("DequantizeLinear", dq_inputs, ["W"], "dequantize", [_attr_int("axis", 0), _attr_int("block_size", block)]),
             _node("MatMul", ["x", "W"], ["y"], "matmul")]
    data = _model("qdq_linear", nodes, inits, [_value_info("x", FLOAT16, (m, k))], [_value_info("y", FLOAT16, (m, n))], opset=21)
    with open(path, "wb") as f:
        f.write(data)
