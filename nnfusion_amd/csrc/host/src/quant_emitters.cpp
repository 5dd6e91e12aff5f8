// Kernel emitters of the quantized operators for ROCM_GPU.  Each emits a host function whose body is
// one call into the gfx950 launcher library (include/nnf_hip_kernels.h) -- the slot where the
// reference's cuda::Dot emits a cuBLAS call (src/nnfusion/core/kernels/cuda_gpu/kernels/dot.cpp:128-205).
// Shapes are written into the body as literals: the code generator de-duplicates kernel definitions by
// signature + body text, so two layers with different N or K must not share a body.
// Registered with TypeConstraint(element::f32) because kernel selection always looks up that key
// (src/nnfusion/engine/pass/graph/kernel_selection.cpp:185-187) and with a priority above every Dot
// emitter of the reference (2); an unsupported node is declined by returning nullptr.
#include "../../nnf_workspace.h"
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
            namespace
            {
                std::string float_literal(double v)
                {
                    std::ostringstream ss;
                    ss << std::scientific << std::setprecision(9) << v << "f";
                    return ss.str();
                }
            } // namespace

            // What the emitters of the quantised products share.
            class QuantLibEmitter : public HipLibEmitter
            {
            public:
                using HipLibEmitter::HipLibEmitter;

            protected:
                // Synchronisation words for the one-launch forms (nnf_plan::sync_flags), when the product of these sizes
                // runs on the tile GEMM or on the row-streaming kernel over ranges of K: a persistent tensor that is zero when the runtime is initialised -- what
                // be_state_buffer is to the reference's BlockFusion kernels
                // (src/nnfusion/engine/pass/graph/blockfusion/blockfusion_codegen.cpp:295-304).  Every launch leaves the
                // words zero again, so one tensor serves all launches of the emitted function.  Returns the statement
                // that declares `name` as the call's nnf_plan, or "" when the product needs none (then pass nullptr).
                std::string declare_sync_plan(const std::string& name, int M, int N, int K, bool gate, bool rms)
                {
                    const nnf::workspace::W4A16Route route =
                        nnf::workspace::route_w4a16(M, N, K, gate, rms, false, nnf::workspace::PLAN_CUS);
                    // (the row-streaming kernel over ranges of K -- a few rows, K above 8192 -- adds its ranges up inside
                    // its launch with one word per workgroup of a range)
                    const bool split = route.kind == nnf::workspace::W4A16Route::MROWS_SPLIT && !gate &&
                                       nnf::workspace::mrows_split_adds_in_launch(N, route.ksplits, nnf::workspace::PLAN_CUS);
                    if (route.kind != nnf::workspace::W4A16Route::TILE && !split)
                        return "";
                    return declare_sync_words(name, split ? nnf::workspace::mrows_split_sync_bytes(nnf::workspace::PLAN_CUS)
                                                          : route.plan.sync_bytes(rms));
                }
                // `name` as an nnf_plan over a persistent, zero-initialised tensor of (at least) `need` bytes; "": none needed
                std::string declare_sync_words(const std::string& name, size_t need)
                {
                    const size_t bytes = (need + 63) & ~(size_t)63;
                    if (bytes == 0 || bytes > NNF_SYNC_FLAGS_BYTES)
                        return "";
                    auto flags = allocate_tensor(Shape{bytes}, element::character, "", ROCM_GPU, true);
                    flags->set_memset(true, 0);
                    std::ostringstream ss;
                    ss << "const nnf_plan " << name << " = {0, 0, 0, " << flags->get_name() << ", " << bytes << ", 0};\n";
                    return ss.str();
                }
            };

            class QuantDot : public QuantLibEmitter
            {
            public:
                explicit QuantDot(std::shared_ptr<KernelContext> ctx)
                    : QuantLibEmitter(ctx)
                {
                }

                LanguageUnit_p emit_function_body() override
                {
                    auto gop = std::dynamic_pointer_cast<op::GenericOp>(m_context->op);
                    if (!gop)
                        return nullptr;
                    auto& cfg = gop->localOpConfig.getRoot();
                    const int group = cfg["group_size"].get<int>();
                    const int zp = cfg["zero_point"].get<int>();
                    const bool rms = cfg["rms_norm"].get<bool>();
                    const bool has_bias = cfg["has_bias"].get<bool>();
                    const bool has_res = cfg["has_residual"].get<bool>();
                    const bool gate = cfg["act"].get<std::string>() == "silu_gate";
                    const int bits = cfg["bits"].get<int>();
                    const bool has_z = cfg["has_zero_points"].get<bool>();
                    // what the launcher supports; anything else is left to other emitters
                    if (!cfg["transpose_B"].get<bool>())
                        return nullptr;
                    if (m_context->inputs[0]->get_element_type() != element::f16 ||
                        m_context->inputs[2]->get_element_type() != element::f16)
                        return nullptr;
                    if (gate && (has_bias || has_res))
                        return nullptr;
                    const Shape& a = m_context->inputs[0]->get_shape();
                    const Shape& w = m_context->inputs[1]->get_shape();
                    const size_t K = a.back();
                    const size_t M = shape_size(a) / K;
                    const size_t N = gate ? w[0] / 2 : w[0];
                    if (M == 0 || N == 0)
                        return nullptr;
                    if (bits != 4 || group != 128 || has_z)
                    {
                        // other block parameters: nnf_wna16_gemm, and for the fused forms nnf_wna16_gemm_fused, which
                        // runs the nodes around the product one after the other (RMSNorm and the product's fp16 output
                        // through scratch memory)
                        if ((bits != 4 && bits != 8) || (group != 32 && group != 64 && group != 128) || K % group != 0 ||
                            (rms && K % 8 != 0))
                            return nullptr;
                        const bool q_fused = rms || has_bias || has_res || gate;
                        // (a residual may turn out to be the output buffer itself: room for the product either way)
                        const size_t q_ws_bytes =
                            q_fused ? nnf::workspace::wna16_fused_layout((int)M, (int)N, (int)K, bits, group, rms, gate, has_res).total()
                                    : nnf::workspace::wna16_gemm((int)M, (int)N, (int)K, bits, group);
                        std::string q_ws = "nullptr";
                        if (q_ws_bytes > 0)
                            q_ws = allocate_tensor(Shape{q_ws_bytes}, element::character)->get_name();
                        size_t qi = 3 + (has_z ? 1 : 0);
                        std::string q_gamma = "nullptr", q_bias = "nullptr", q_res = "nullptr";
                        if (rms)
                            q_gamma = "input" + std::to_string(qi++);
                        if (has_bias)
                            q_bias = "input" + std::to_string(qi++);
                        if (has_res)
                            q_res = "input" + std::to_string(qi++);
                        LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                        *lu << "const nnf_quant quant = {" << bits << ", " << group << ", " << zp << ", "
                            << (has_z ? "input3" : "nullptr") << "};\n";
                        // 4-bit weights on the stream-K tile GEMM (above 16 rows, K a multiple of 256): its synchronisation words
                        std::string q_plan;
                        if (!q_fused && bits == 4 && M > 16 && nnf::workspace::w4a16_gemm_q_fits((int)M, (int)N, (int)K, group == 32 ? 5 : group == 64 ? 6 : 7))
                            q_plan = declare_sync_words("plan", nnf::workspace::plan_w4a16_sk((int)M, (int)N, (int)K, false, nnf::workspace::PLAN_CUS).sync_bytes());
                        *lu << q_plan;
                        if (!q_fused && !q_plan.empty())
                            *lu << "NNF_HIP_CHECK(nnf_wna16_gemm_planned(stream, input0, input1, input2, output0, " << M << ", " << N << ", "
                                << K << ", &quant, &plan, " << q_ws << ", " << q_ws_bytes << "));\n";
                        else if (!q_fused)
                            *lu << "NNF_HIP_CHECK(nnf_wna16_gemm(stream, input0, input1, input2, output0, " << M << ", " << N << ", "
                                << K << ", &quant, " << q_ws << ", " << q_ws_bytes << "));\n";
                        else
                            *lu << "NNF_HIP_CHECK(nnf_wna16_gemm_fused(stream, input0, input1, input2, output0, " << M << ", " << N
                                << ", " << K << ", &quant, " << q_gamma << ", " << float_literal(cfg["rms_eps"].get<double>()) << ", "
                                << q_bias << ", " << q_res << ", " << (gate ? "NNF_ACT_SILU_GATE" : "NNF_ACT_NONE") << ", " << q_ws
                                << ", " << q_ws_bytes << "));\n";
                        return lu;
                    }
                    if (K % 128 != 0)
                        return nullptr;

                    size_t idx = 3;
                    std::string gamma = "nullptr", bias = "nullptr", residual = "nullptr";
                    if (rms)
                        gamma = "input" + std::to_string(idx++);
                    if (has_bias)
                        bias = "input" + std::to_string(idx++);
                    if (has_res)
                        residual = "input" + std::to_string(idx++);

                    const bool fused = rms || has_bias || has_res || gate;
                    const size_t ws_bytes = fused ? nnf::workspace::w4a16_gemm_fused((int)M, (int)N, (int)K, group, gate)
                                                  : nnf::workspace::w4a16_gemm((int)M, (int)N, (int)K, group);
                    std::string ws = "nullptr";
                    if (ws_bytes > 0)
                        ws = allocate_tensor(Shape{ws_bytes}, element::character)->get_name();

                    // the tile GEMM in one launch (ahead of the body's text: the tensor is part of the kernel's context)
                    const std::string plan = declare_sync_plan("plan", (int)M, (int)N, (int)K, gate, rms);
                    LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                    *lu << plan;
                    if (!fused && plan.empty())
                    {
                        *lu << "NNF_HIP_CHECK(nnf_w4a16_gemm(stream, input0, input1, input2, output0, " << M << ", " << N
                            << ", " << K << ", " << group << ", " << zp << ", " << ws << ", " << ws_bytes << "));\n";
                    }
                    else if (!fused)
                    {
                        *lu << "NNF_HIP_CHECK(nnf_w4a16_gemm_variant(stream, input0, input1, input2, output0, " << M << ", " << N
                            << ", " << K << ", " << group << ", " << zp << ", NNF_W4A16_AUTO, &plan, " << ws << ", " << ws_bytes
                            << "));\n";
                    }
                    else
                    {
                        *lu << "NNF_HIP_CHECK(nnf_w4a16_gemm_fused_variant(stream, input0, input1, input2, output0, " << M << ", "
                            << N << ", " << K << ", " << group << ", " << zp << ", " << gamma << ", "
                            << float_literal(cfg["rms_eps"].get<double>()) << ", " << bias << ", " << residual << ", "
                            << (gate ? "NNF_ACT_SILU_GATE" : "NNF_ACT_NONE") << ", NNF_W4A16_AUTO, "
                            << (plan.empty() ? "nullptr" : "&plan") << ", " << ws << ", " << ws_bytes << "));\n";
                    }
                    return lu;
                }
            };

            // One kernel variant of the plain fp16 x int4 product (no fused prologue / epilogue): the emitters
            // that ProfilingBasedKernelSelector times against the automatic one.  A variant that cannot serve
            // the node's shape declines it.
            template <int VARIANT>
            class QuantDotVariant : public HipLibEmitter
            {
            public:
                explicit QuantDotVariant(std::shared_ptr<KernelContext> ctx)
                    : HipLibEmitter(ctx, std::string("rocm_") + variant_name())
                {
                }
                static const char* variant_name()
                {
                    return VARIANT == 1 ? "gemv_valu" : VARIANT == 2 ? "gemv_mfma" : VARIANT == 3 ? "gemm_mfma" : "gemv_rows";
                }
                static const char* variant_enum()
                {
                    return VARIANT == 1 ? "NNF_W4A16_GEMV_VALU"
                                        : VARIANT == 2 ? "NNF_W4A16_GEMV_MFMA"
                                                       : VARIANT == 3 ? "NNF_W4A16_GEMM_MFMA" : "NNF_W4A16_GEMV_ROWS";
                }

                LanguageUnit_p emit_function_body() override
                {
                    auto gop = std::dynamic_pointer_cast<op::GenericOp>(m_context->op);
                    if (!gop)
                        return nullptr;
                    auto& cfg = gop->localOpConfig.getRoot();
                    const int group = cfg["group_size"].get<int>();
                    const int zp = cfg["zero_point"].get<int>();
                    if (cfg["rms_norm"].get<bool>() || cfg["has_bias"].get<bool>() || cfg["has_residual"].get<bool>() ||
                        cfg["act"].get<std::string>() == "silu_gate")
                        return nullptr;
                    if (cfg["bits"].get<int>() != 4 || group != 128 || cfg["has_zero_points"].get<bool>() ||
                        !cfg["transpose_B"].get<bool>())
                        return nullptr;
                    if (m_context->inputs[0]->get_element_type() != element::f16 ||
                        m_context->inputs[2]->get_element_type() != element::f16)
                        return nullptr;
                    const Shape& a = m_context->inputs[0]->get_shape();
                    const Shape& w = m_context->inputs[1]->get_shape();
                    const size_t K = a.back();
                    const size_t M = shape_size(a) / K;
                    const size_t N = w[0];
                    if (!nnf::workspace::w4a16_variant_fits((int)M, (int)N, (int)K, VARIANT))
                        return nullptr;
                    // partial sums of the tile GEMM (tiles shared by several workgroups) or of a GEMV kernel over ranges of K
                    const size_t ws_bytes = VARIANT == 1 ? 0
                                                         : nnf::workspace::route_w4a16((int)M, (int)N, (int)K, false, false, false,
                                                                                       nnf::workspace::PLAN_CUS, VARIANT)
                                                               .partial_bytes;
                    std::string ws = "nullptr";
                    if (ws_bytes > 0)
                        ws = allocate_tensor(Shape{ws_bytes}, element::character)->get_name();
                    LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                    *lu << "NNF_HIP_CHECK(nnf_w4a16_gemm_variant(stream, input0, input1, input2, output0, " << M << ", " << N
                        << ", " << K << ", " << group << ", " << zp << ", " << variant_enum() << ", nullptr, " << ws << ", "
                        << ws_bytes << "));\n";
                    return lu;
                }
            };

            class QuantDotW8A8 : public QuantLibEmitter
            {
            public:
                explicit QuantDotW8A8(std::shared_ptr<KernelContext> ctx)
                    : QuantLibEmitter(ctx)
                {
                }

                LanguageUnit_p emit_function_body() override
                {
                    auto gop = std::dynamic_pointer_cast<op::GenericOp>(m_context->op);
                    if (!gop)
                        return nullptr;
                    const Shape& a = m_context->inputs[0]->get_shape();
                    const Shape& w = m_context->inputs[2]->get_shape();
                    const size_t M = a[0], K = a[1], N = w[0];
                    if (K % 128 != 0 || K > 133000 || M == 0 || N == 0)
                        return nullptr;
                    const bool raw = gop->localOpConfig.getRoot()["out_type"].get<std::string>() == "i32";
                    // int32 partial sums when the tile plan of the shape splits K
                    const size_t ws_bytes = nnf::workspace::w8a8_gemm((int)M, (int)N, (int)K);
                    std::string ws = "nullptr";
                    if (ws_bytes > 0)
                        ws = allocate_tensor(Shape{ws_bytes}, element::character)->get_name();
                    // a few rows with a long K: the row-streaming kernel over two ranges of K, which meet at one word per
                    // workgroup of a range
                    std::string plan;
                    if (nnf::workspace::w8a8_mrows_preferred((int)M, (int)N, (int)K, nnf::workspace::PLAN_CUS) &&
                        nnf::workspace::w8a8_mrows_ranges((int)M, (int)N, (int)K, nnf::workspace::PLAN_CUS) > 1)
                        plan = declare_sync_words("plan", nnf::workspace::mrows_split_sync_bytes(nnf::workspace::PLAN_CUS));
                    LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                    *lu << plan;
                    if (!plan.empty())
                        *lu << "NNF_HIP_CHECK(nnf_w8a8_gemm_variant(stream, input0, " << (raw ? "nullptr" : "input1") << ", input2, "
                            << (raw ? "nullptr" : "input3") << ", " << (raw ? "nullptr, output0" : "output0, nullptr") << ", " << M
                            << ", " << N << ", " << K << ", NNF_W8A8_AUTO, &plan, " << ws << ", " << ws_bytes << "));\n";
                    else if (raw)
                        *lu << "NNF_HIP_CHECK(nnf_w8a8_gemm_acc(stream, input0, input2, output0, " << M << ", " << N << ", "
                            << K << ", " << ws << ", " << ws_bytes << "));\n";
                    else
                        *lu << "NNF_HIP_CHECK(nnf_w8a8_gemm(stream, input0, input1, input2, input3, output0, " << M << ", "
                            << N << ", " << K << ", " << ws << ", " << ws_bytes << "));\n";
                    return lu;
                }
            };

            class FusedQuantMLP : public QuantLibEmitter
            {
            public:
                explicit FusedQuantMLP(std::shared_ptr<KernelContext> ctx)
                    : QuantLibEmitter(ctx)
                {
                }

                LanguageUnit_p emit_function_body() override
                {
                    auto gop = std::dynamic_pointer_cast<op::GenericOp>(m_context->op);
                    if (!gop)
                        return nullptr;
                    auto& cfg = gop->localOpConfig.getRoot();
                    const int group = cfg["group_size"].get<int>();
                    const int zp = cfg["zero_point"].get<int>();
                    const Shape& x = m_context->inputs[0]->get_shape();
                    const size_t M = x[0], H = x[1], I = m_context->inputs[2]->get_shape()[0] / 2;
                    const int bits = cfg["bits"].get<int>();
                    const int zp_down = cfg["zero_point_down"].get<int>() < 0 ? zp : cfg["zero_point_down"].get<int>();
                    const bool z_gu = cfg["has_zero_points_gate_up"].get<bool>(), z_d = cfg["has_zero_points_down"].get<bool>();
                    if (bits != 4 || group != 128 || z_gu || z_d || zp_down != zp)
                    {
                        // other block parameters: the nodes of the block one after the other inside one call
                        if ((bits != 4 && bits != 8) || (group != 32 && group != 64 && group != 128) || H % group != 0 || I % group != 0 ||
                            H % 8 != 0 || M == 0)
                            return nullptr;
                        const size_t q_bytes = nnf::workspace::fused_mlp_wna16((int)M, (int)H, (int)I, bits, group);
                        auto q_ws = allocate_tensor(Shape{q_bytes}, element::character);
                        size_t zi = 6;
                        const std::string zgu = z_gu ? "input" + std::to_string(zi++) : "nullptr";
                        const std::string zd = z_d ? "input" + std::to_string(zi++) : "nullptr";
                        LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                        *lu << "const nnf_quant quant_gate_up = {" << bits << ", " << group << ", " << zp << ", " << zgu << "};\n";
                        *lu << "const nnf_quant quant_down = {" << bits << ", " << group << ", " << zp_down << ", " << zd << "};\n";
                        *lu << "NNF_HIP_CHECK(nnf_fused_mlp_wna16(stream, input0, input1, " << float_literal(cfg["rms_eps"].get<double>())
                            << ", input2, input3, input4, input5, output0, " << M << ", " << H << ", " << I
                            << ", &quant_gate_up, &quant_down, " << q_ws->get_name() << ", " << q_bytes << "));\n";
                        return lu;
                    }
                    if (H % 128 != 0 || I % 128 != 0 || M == 0)
                        return nullptr;
                    const size_t ws_bytes = nnf::workspace::fused_mlp_w4a16((int)M, (int)H, (int)I, group);
                    // the only intermediate that reaches HBM: h [M, I] fp16 (plus M row statistics)
                    auto ws = allocate_tensor(Shape{ws_bytes}, element::character);
                    // either product on the tile GEMM: in one launch each
                    const std::string plan_gu = declare_sync_plan("gate_up_plan", (int)M, (int)I, (int)H, true, true);
                    const std::string plan_d = declare_sync_plan("down_plan", (int)M, (int)H, (int)I, false, false);
                    LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                    *lu << plan_gu << plan_d;
                    *lu << "NNF_HIP_CHECK(nnf_fused_mlp_w4a16_planned(stream, input0, input1, "
                        << float_literal(cfg["rms_eps"].get<double>()) << ", input2, input3, input4, input5, output0, " << M
                        << ", " << H << ", " << I << ", " << group << ", " << zp << ", "
                        << (plan_gu.empty() ? "nullptr" : "&gate_up_plan") << ", " << (plan_d.empty() ? "nullptr" : "&down_plan")
                        << ", " << ws->get_name() << ", " << ws_bytes << "));\n";
                    return lu;
                }
            };

            // Slice of the last axis (what QuantGemmFusionPass puts behind a merged QuantDot): a strided
            // device-to-device copy, no kernel of its own.
            class Slice : public HipLibEmitter
            {
            public:
                explicit Slice(std::shared_ptr<KernelContext> ctx)
                    : HipLibEmitter(ctx)
                {
                }

                LanguageUnit_p emit_function_body() override
                {
                    auto gop = std::dynamic_pointer_cast<op::GenericOp>(m_context->op);
                    if (!gop)
                        return nullptr;
                    const Shape& in = m_context->inputs[0]->get_shape();
                    const Shape& out = m_context->outputs[0]->get_shape();
                    if (in.empty() || in.size() != out.size())
                        return nullptr;
                    const size_t elt = m_context->inputs[0]->get_element_type().size();
                    const size_t rows = shape_size(in) / in.back();
                    const size_t begin = (size_t)gop->localOpConfig.getRoot()["begin"].get<int>();
                    LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                    *lu << "HIP_SAFE_CALL(hipMemcpy2DAsync(output0, " << out.back() * elt << ", (const char*)input0 + "
                        << begin * elt << ", " << in.back() * elt << ", " << out.back() * elt << ", " << rows
                        << ", hipMemcpyDeviceToDevice, stream));\n";
                    return lu;
                }

                LanguageUnit_p emit_dependency() override
                {
                    LanguageUnit_p lu = HipLibEmitter::emit_dependency();
                    lu->require(macro::HIP_SAFE_CALL);
                    return lu;
                }
            };
        } // namespace hip

        REGISTER_KERNEL_EMITTER("Slice", Device(ROCM_GPU).TypeConstraint(element::f32).Tag("nnf_hip_gfx950").Priority(5),
                                hip::Slice)
        REGISTER_KERNEL_EMITTER("QuantDot",
                                Device(ROCM_GPU).TypeConstraint(element::f32).Tag("nnf_hip_gfx950").Priority(5),
                                hip::QuantDot)
        // the variants rank below the automatic emitter (DefaultKernelSelector keeps picking that one) and above
        // the reference's Dot emitters
        REGISTER_KERNEL_EMITTER("QuantDot",
                                Device(ROCM_GPU).TypeConstraint(element::f32).Tag("nnf_hip_gfx950_gemv_rows").Priority(3),
                                hip::QuantDotVariant<4>)
        REGISTER_KERNEL_EMITTER("QuantDot",
                                Device(ROCM_GPU).TypeConstraint(element::f32).Tag("nnf_hip_gfx950_gemv_mfma").Priority(3),
                                hip::QuantDotVariant<2>)
        REGISTER_KERNEL_EMITTER("QuantDot",
                                Device(ROCM_GPU).TypeConstraint(element::f32).Tag("nnf_hip_gfx950_gemm_mfma").Priority(3),
                                hip::QuantDotVariant<3>)
        REGISTER_KERNEL_EMITTER("QuantDot",
                                Device(ROCM_GPU).TypeConstraint(element::f32).Tag("nnf_hip_gfx950_gemv_valu").Priority(3),
                                hip::QuantDotVariant<1>)
        REGISTER_KERNEL_EMITTER("QuantDotW8A8",
                                Device(ROCM_GPU).TypeConstraint(element::f32).Tag("nnf_hip_gfx950").Priority(5),
                                hip::QuantDotW8A8)
        REGISTER_KERNEL_EMITTER("FusedQuantMLP",
                                Device(ROCM_GPU).TypeConstraint(element::f32).Tag("nnf_hip_gfx950").Priority(5),
                                hip::FusedQuantMLP)
    } // namespace kernels
} // namespace nnfusion
