// Kernel emitters for the nodes AROUND a quantized product -- RMSNorm, Add, Multiply, Sigmoid, Swish, Dequantize -- for
// graphs in which the fusion passes left some of them standing (a gate product with a second consumer, a normalisation
// that feeds something else as well, a Dequantize that does not feed a product).  Without them such a node stops code
// generation: the reference compiles these graphs through its element-wise emitter
// (src/nnfusion/core/kernels/cuda_gpu/kernels/elementwise.cpp over the CudaOpMap entries of
// cuda_gpu/cuda_kernelops.hpp:408 Add, :416 Multiply, :447-451 Sigmoid) and layer_norm.cpp.  Each emits a host function
// around one call into the launcher library, like the emitters of the products (quant_emitters.cpp).
#include "nnf_hip_kernels.h"
#include "nnfusion/core/kernels/hip_gpu/hip_emitter.hpp"
#include "nnfusion/core/kernels/kernel_registration.hpp"
#include "nnfusion/core/operators/generic_op/generic_op.hpp"

#include <iomanip>

namespace nnfusion
{
    namespace kernels
    {
        namespace hip
        {
            // Add / Multiply (two operands of one shape, or one of them a row [cols] broadcast over the other's leading
            // axes) and the unary Sigmoid / Swish, on fp16 tensors
            template <int OP>
            class Elementwise : public HipLibEmitter
            {
            public:
                explicit Elementwise(std::shared_ptr<KernelContext> ctx)
                    : HipLibEmitter(ctx)
                {
                }
                static const char* op_enum()
                {
                    return OP == NNF_EW_ADD ? "NNF_EW_ADD" : OP == NNF_EW_MULTIPLY ? "NNF_EW_MULTIPLY" : OP == NNF_EW_SIGMOID ? "NNF_EW_SIGMOID" : "NNF_EW_SWISH";
                }

                LanguageUnit_p emit_function_body() override
                {
                    constexpr bool binary = OP == NNF_EW_ADD || OP == NNF_EW_MULTIPLY;
                    if (m_context->inputs.size() != (binary ? 2u : 1u) || m_context->outputs.size() != 1)
                        return nullptr;
                    for (auto& t : m_context->inputs)
                        if (t->get_element_type() != element::f16)
                            return nullptr;
                    const Shape& out = m_context->outputs[0]->get_shape();
                    if (out.empty() || shape_size(out) == 0)
                        return nullptr;
                    const size_t cols = out.back(), rows = shape_size(out) / cols;
                    std::string a = "input0", b = "nullptr";
                    bool b_is_row = false;
                    if (binary)
                    {
                        // the full-size operand first; the other one the same shape, or a row
                        const Shape& s0 = m_context->inputs[0]->get_shape();
                        const Shape& s1 = m_context->inputs[1]->get_shape();
                        const bool first_full = s0 == out, second_full = s1 == out;
                        if (!first_full && !second_full)
                            return nullptr;
                        a = first_full ? "input0" : "input1";
                        b = first_full ? "input1" : "input0";
                        const Shape& other = first_full ? s1 : s0;
                        if (other != out)
                        {
                            if (other.size() != 1 || other[0] != cols)
                                return nullptr;
                            b_is_row = true;
                        }
                    }
                    LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                    *lu << "NNF_HIP_CHECK(nnf_elementwise_f16(stream, " << op_enum() << ", " << a << ", " << b << ", output0, " << rows
                        << ", " << cols << ", " << (b_is_row ? 1 : 0) << "));\n";
                    return lu;
                }
            };

            class RMSNorm : public HipLibEmitter
            {
            public:
                explicit RMSNorm(std::shared_ptr<KernelContext> ctx)
                    : HipLibEmitter(ctx)
                {
                }
                LanguageUnit_p emit_function_body() override
                {
                    auto gop = std::dynamic_pointer_cast<op::GenericOp>(m_context->op);
                    if (!gop || m_context->inputs.size() != 2 || m_context->inputs[0]->get_element_type() != element::f16 ||
                        m_context->inputs[1]->get_element_type() != element::f16)
                        return nullptr;
                    const Shape& x = m_context->inputs[0]->get_shape();
                    if (x.empty() || x.back() % 8 != 0 || shape_size(x) == 0)
                        return nullptr;
                    std::ostringstream eps;
                    eps << std::scientific << std::setprecision(9) << gop->localOpConfig.getRoot()["eps"].get<double>() << "f";
                    LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                    *lu << "NNF_HIP_CHECK(nnf_rms_norm_f16(stream, input0, input1, output0, " << shape_size(x) / x.back() << ", " << x.back()
                        << ", " << eps.str() << "));\n";
                    return lu;
                }
            };

            // Dequantize of block-quantized weights (the inputs and attributes of QuantDot's weight side)
            class Dequantize : public HipLibEmitter
            {
            public:
                explicit Dequantize(std::shared_ptr<KernelContext> ctx)
                    : HipLibEmitter(ctx)
                {
                }
                LanguageUnit_p emit_function_body() override
                {
                    auto gop = std::dynamic_pointer_cast<op::GenericOp>(m_context->op);
                    if (!gop)
                        return nullptr;
                    auto& cfg = gop->localOpConfig.getRoot();
                    const int bits = cfg["bits"].get<int>(), group = cfg["group_size"].get<int>(), zp = cfg["zero_point"].get<int>();
                    const bool has_z = cfg["has_zero_points"].get<bool>();
                    const Shape& out = m_context->outputs[0]->get_shape();
                    if ((bits != 4 && bits != 8) || (group != 32 && group != 64 && group != 128) || out.size() != 2 ||
                        out[1] % (size_t)group != 0 || m_context->outputs[0]->get_element_type() != element::f16 ||
                        m_context->inputs[1]->get_element_type() != element::f16)
                        return nullptr;
                    LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                    *lu << "const nnf_quant quant = {" << bits << ", " << group << ", " << zp << ", " << (has_z ? "input2" : "nullptr")
                        << "};\n";
                    *lu << "NNF_HIP_CHECK(nnf_dequantize_f16(stream, input0, input1, output0, " << out[0] << ", " << out[1]
                        << ", &quant));\n";
                    return lu;
                }
            };
        } // namespace hip

#define NNF_REGISTER_NODE(OPNAME, CLASS)                                                                                          \
    REGISTER_KERNEL_EMITTER(OPNAME, Device(ROCM_GPU).TypeConstraint(element::f32).Tag("nnf_hip_gfx950").Priority(5), CLASS)
        NNF_REGISTER_NODE("Add", hip::Elementwise<NNF_EW_ADD>)
        NNF_REGISTER_NODE("Multiply", hip::Elementwise<NNF_EW_MULTIPLY>)
        NNF_REGISTER_NODE("Sigmoid", hip::Elementwise<NNF_EW_SIGMOID>)
        NNF_REGISTER_NODE("Swish", hip::Elementwise<NNF_EW_SWISH>)
        NNF_REGISTER_NODE("RMSNorm", hip::RMSNorm)
        NNF_REGISTER_NODE("Dequantize", hip::Dequantize)
#undef NNF_REGISTER_NODE
    } // namespace kernels
} // namespace nnfusion
