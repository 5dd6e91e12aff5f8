// The quantized operators, declared through the operator-plugin interface (REGISTER_OP / GenericOp,
// precedent: src/nnfusion/core/operators/generic_op/generic_op_define/MatMulAdd.cpp:6-35).
// They are GenericOps, not op::Dot: Dot's validation merges the element types of its two inputs and
// rejects fp16 x u8 (src/nnfusion/core/operators/op_define/dot.cpp:47-53).
//
//   QuantDot       inputs: A f16 [M,K], Wq u8 [N,K*bits/8] (bits 4: two per byte, low nibble first), S f16 [N,K/group]
//                          [, Z u8 [N, ceil(K/group*bits/8)]] [, gamma f16 [K]] [, bias f16 [N]] [, residual f16 [M,N]]
//                          (in this order, by attribute; Z: one zero point per (row, group), 4-bit ones two per byte)
//                  attrs : bits 4|8, group_size 128, zero_point 8 (scalar, when has_zero_points is false), transpose_B true,
//                          has_zero_points false,
//                          rms_norm false, rms_eps 1e-6, has_bias false, has_residual false, act "none"|"silu_gate"
//                  output: Y f16 [M, N]   (N = rows of Wq; half of them when act == "silu_gate")
//   QuantDotW8A8   inputs: A i8 [M,K], s_tok f32 [M], W i8 [N,K], s_ch f32 [N];  attr out_type "f16"|"i32"
//                  output: Y f16 [M,N] = fp16((float)acc * s_tok * s_ch), or the raw i32 accumulators
//   FusedQuantMLP  inputs: x f16 [M,H], gamma f16 [H], Wgu u8 [2I,H*bits/8], Sgu f16 [2I,H/g], Wd u8 [H,I*bits/8], Sd f16 [H,I/g]
//                          [, Zgu u8] [, Zd u8] (zero points per (row, group) of either matrix, by attribute)
//                  attrs : bits 4, group_size 128, zero_point 8, zero_point_down -1 (= zero_point), has_zero_points_gate_up false,
//                          has_zero_points_down false, rms_eps 1e-6
//                  output: out f16 [M,H] = x + Wd . (SiLU(Wg . n) * (Wu . n)), n = RMSNorm(x)
#include "nnfusion/core/operators/generic_op/generic_op.hpp"

using namespace nnfusion;

namespace
{
    int int_attr(std::shared_ptr<op::GenericOp> gop, const std::string& key)
    {
        return gop->localOpConfig.getRoot()[key].get<int>();
    }
    bool bool_attr(std::shared_ptr<op::GenericOp> gop, const std::string& key)
    {
        return gop->localOpConfig.getRoot()[key].get<bool>();
    }
} // namespace

REGISTER_OP(QuantDot)
    .attr<int>("bits", 4)
    .attr<int>("group_size", 128)
    .attr<int>("zero_point", 8)
    .attr<bool>("transpose_B", true)
    .attr<bool>("has_zero_points", false)
    .attr<bool>("rms_norm", false)
    .attr<double>("rms_eps", 1e-6)
    .attr<bool>("has_bias", false)
    .attr<bool>("has_residual", false)
    .attr<std::string>("act", "none")
    .constrait([](const op::OpConfig::any& config) -> bool {
        const int bits = config.at("bits").get<int>();
        if (bits != 4 && bits != 8)
            return false;
        int zp = config.at("zero_point").get<int>();
        if (zp < 0 || zp >= (1 << bits) || config.at("group_size").get<int>() <= 0)
            return false;
        auto act = config.at("act").get<std::string>();
        return act == "none" || act == "silu_gate";
    })
    .infershape([](std::shared_ptr<graph::GNode> gnode) -> void {
        auto gop = std::dynamic_pointer_cast<op::GenericOp>(gnode->get_op_ptr());
        NNFUSION_CHECK_NOT_NULLPTR(gop);
        const bool has_z = bool_attr(gop, "has_zero_points");
        size_t expect = 3 + (has_z ? 1 : 0) + (bool_attr(gop, "rms_norm") ? 1 : 0) + (bool_attr(gop, "has_bias") ? 1 : 0) +
                        (bool_attr(gop, "has_residual") ? 1 : 0);
        OP_VALIDATION(gop, gnode->get_input_size() == expect) << "expected " << expect << " inputs";
        const Shape& a = gnode->get_input_shape(0);
        const Shape& w = gnode->get_input_shape(1);
        const Shape& s = gnode->get_input_shape(2);
        OP_VALIDATION(gop, a.size() >= 1 && w.size() == 2 && s.size() == 2) << "bad ranks";
        OP_VALIDATION(gop, gnode->get_input_element_type(1) == element::u8) << "quantized weights travel as u8";
        const size_t K = a.back();
        const size_t group = (size_t)int_attr(gop, "group_size");
        const size_t bits = (size_t)int_attr(gop, "bits");
        OP_VALIDATION(gop, w[1] * 8 == K * bits) << "Wq must be [N, K*bits/8]";
        OP_VALIDATION(gop, K % group == 0 && s[0] == w[0] && s[1] == K / group) << "scales must be [N, K/group]";
        if (has_z)
        {
            const Shape& z = gnode->get_input_shape(3);
            OP_VALIDATION(gop, gnode->get_input_element_type(3) == element::u8 && z.size() == 2 && z[0] == w[0] &&
                                   z[1] == (K / group * bits + 7) / 8)
                << "zero points must be u8 [N, ceil(K/group*bits/8)]";
        }
        size_t N = w[0];
        if (gop->localOpConfig.getRoot()["act"].get<std::string>() == "silu_gate")
        {
            OP_VALIDATION(gop, N % 2 == 0) << "gate|up weights need an even row count";
            N /= 2;
        }
        Shape out(a.begin(), a.end() - 1);
        out.push_back(N);
        gnode->set_output_type_and_shape(0, gnode->get_input_element_type(0), out);
    });

REGISTER_OP(QuantDotW8A8)
    .attr<std::string>("out_type", "f16")
    .constrait([](const op::OpConfig::any& config) -> bool {
        auto t = config.at("out_type").get<std::string>();
        return t == "f16" || t == "i32";
    })
    .infershape([](std::shared_ptr<graph::GNode> gnode) -> void {
        auto gop = std::dynamic_pointer_cast<op::GenericOp>(gnode->get_op_ptr());
        NNFUSION_CHECK_NOT_NULLPTR(gop);
        OP_VALIDATION(gop, gnode->get_input_size() == 4) << "inputs: A, s_tok, W, s_ch";
        const Shape& a = gnode->get_input_shape(0);
        const Shape& w = gnode->get_input_shape(2);
        OP_VALIDATION(gop, a.size() == 2 && w.size() == 2 && a[1] == w[1]) << "A [M,K], W [N,K]";
        OP_VALIDATION(gop, gnode->get_input_element_type(0) == element::i8 &&
                               gnode->get_input_element_type(2) == element::i8)
            << "int8 operands";
        OP_VALIDATION(gop, shape_size(gnode->get_input_shape(1)) == a[0] && shape_size(gnode->get_input_shape(3)) == w[0])
            << "one scale per token and per output channel";
        bool raw = gop->localOpConfig.getRoot()["out_type"].get<std::string>() == "i32";
        gnode->set_output_type_and_shape(0, raw ? element::i32 : element::f16, Shape{a[0], w[0]});
    });

REGISTER_OP(FusedQuantMLP)
    .attr<int>("bits", 4)
    .attr<int>("group_size", 128)
    .attr<int>("zero_point", 8)
    .attr<int>("zero_point_down", -1) // -1: the same as zero_point
    .attr<bool>("has_zero_points_gate_up", false)
    .attr<bool>("has_zero_points_down", false)
    .attr<double>("rms_eps", 1e-6)
    .infershape([](std::shared_ptr<graph::GNode> gnode) -> void {
        auto gop = std::dynamic_pointer_cast<op::GenericOp>(gnode->get_op_ptr());
        NNFUSION_CHECK_NOT_NULLPTR(gop);
        const size_t expect = 6 + (bool_attr(gop, "has_zero_points_gate_up") ? 1 : 0) + (bool_attr(gop, "has_zero_points_down") ? 1 : 0);
        OP_VALIDATION(gop, gnode->get_input_size() == expect) << "inputs: x, gamma, Wgu, Sgu, Wd, Sd [, Zgu] [, Zd]";
        const Shape& x = gnode->get_input_shape(0);
        const Shape& wgu = gnode->get_input_shape(2);
        const Shape& wd = gnode->get_input_shape(4);
        OP_VALIDATION(gop, x.size() == 2 && wgu.size() == 2 && wd.size() == 2) << "bad ranks";
        const size_t bits = (size_t)int_attr(gop, "bits");
        OP_VALIDATION(gop, bits == 4 || bits == 8) << "4- or 8-bit weights";
        const size_t H = x[1], I = wgu[0] / 2;
        OP_VALIDATION(gop, wgu[1] * 8 == H * bits && wd[0] == H && wd[1] * 8 == I * bits && wgu[0] % 2 == 0) << "shape mismatch";
        gnode->set_output_type_and_shape(0, gnode->get_input_element_type(0), x);
    });

// Dequantize of block-quantized weights: the reference's Dequantize (core/operators/op_define/dequantize.hpp; arithmetic
// core/kernels/cpu/reference/kernels.cpp:601-623) with scales and offsets per block of `group_size` weights along K.
//   inputs: Wq u8 [N, K*bits/8], S f16 [N, K/group] [, Z u8 [N, ceil(K/group*bits/8)]]   output: W f16 [N, K]
REGISTER_OP(Dequantize)
    .attr<int>("bits", 4)
    .attr<int>("group_size", 128)
    .attr<int>("zero_point", 8)
    .attr<bool>("has_zero_points", false)
    .infershape([](std::shared_ptr<graph::GNode> gnode) -> void {
        auto gop = std::dynamic_pointer_cast<op::GenericOp>(gnode->get_op_ptr());
        NNFUSION_CHECK_NOT_NULLPTR(gop);
        const bool has_z = bool_attr(gop, "has_zero_points");
        OP_VALIDATION(gop, gnode->get_input_size() == (has_z ? 3u : 2u)) << "inputs: Wq, S [, Z]";
        const Shape& w = gnode->get_input_shape(0);
        const Shape& s = gnode->get_input_shape(1);
        const size_t bits = (size_t)int_attr(gop, "bits"), group = (size_t)int_attr(gop, "group_size");
        OP_VALIDATION(gop, w.size() == 2 && s.size() == 2 && (bits == 4 || bits == 8) && group > 0) << "bad ranks or attributes";
        const size_t K = w[1] * 8 / bits;
        OP_VALIDATION(gop, K % group == 0 && s[0] == w[0] && s[1] == K / group) << "scales must be [N, K/group]";
        gnode->set_output_type_and_shape(0, gnode->get_input_element_type(1), Shape{w[0], K});
    });

// The unquantized product, as far as the fold into QuantDot needs it: one reduction axis, A [.., K] . B [K, N] or (transpose_B)
// B [N, K]; operands of one element type (src/nnfusion/core/operators/op_define/dot.cpp:47-53, 116-125).
REGISTER_OP(Dot)
    .attr<bool>("transpose_A", false)
    .attr<bool>("transpose_B", false)
    .infershape([](std::shared_ptr<graph::GNode> gnode) -> void {
        auto gop = std::dynamic_pointer_cast<op::GenericOp>(gnode->get_op_ptr());
        NNFUSION_CHECK_NOT_NULLPTR(gop);
        OP_VALIDATION(gop, gnode->get_input_size() == 2) << "two inputs";
        OP_VALIDATION(gop, gnode->get_input_element_type(0) == gnode->get_input_element_type(1)) << "arguments do not have the same element type";
        OP_VALIDATION(gop, !bool_attr(gop, "transpose_A")) << "transpose_A is not supported";
        const Shape& a = gnode->get_input_shape(0);
        const Shape& b = gnode->get_input_shape(1);
        OP_VALIDATION(gop, a.size() >= 1 && b.size() == 2) << "bad ranks";
        const bool tb = bool_attr(gop, "transpose_B");
        OP_VALIDATION(gop, a.back() == (tb ? b[1] : b[0])) << "reduction axes do not match";
        Shape out(a.begin(), a.end() - 1);
        out.push_back(tb ? b[0] : b[1]);
        gnode->set_output_type_and_shape(0, gnode->get_input_element_type(0), out);
    });
