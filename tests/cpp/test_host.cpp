// Host-side unit tests (no GPU): the kernel plugin API restated from the reference -- registry,
// selection order, decline-by-nullptr, naming, the f32 lookup key -- exercised with fake emitters, the
// quantized operators' shape inference, the text the quantized emitters produce, the code generator's
// hook order and output, and the single-kernel harness source.  Run by tests/test_host_cpp.py; prints one
// line per case and exits non-zero on the first failure of any case.
#include "nnfusion/core/kernels/hip_gpu/hip_emitter.hpp"
#include "nnfusion/core/kernels/kernel_registration.hpp"
#include "nnfusion/core/operators/generic_op/generic_op.hpp"
#include "nnfusion/engine/pass/codegen/base_codegen_pass.hpp"
#include "nnfusion/engine/pass/graph/kernel_selection.hpp"
#include "nnfusion/engine/pass/graph/quant_fusion_pass.hpp"
#include "nnfusion/engine/profiler/hip_runtime.hpp"
#include "nnfusion/frontend/onnx_import/onnx.hpp"

#include <algorithm>

#include "../../nnfusion_amd/csrc/nnf_workspace.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iterator>

using namespace nnfusion;
using namespace nnfusion::kernels;

static int g_failures = 0;
static std::string g_case;

#define EXPECT(cond)                                                                                           \
    do                                                                                                         \
    {                                                                                                          \
        if (!(cond))                                                                                           \
        {                                                                                                      \
            printf("FAIL %s: %s (line %d)\n", g_case.c_str(), #cond, __LINE__);                                \
            ++g_failures;                                                                                      \
        }                                                                                                      \
    } while (0)

#define CONTAINS(text, needle) EXPECT((text).find(needle) != std::string::npos)

template <typename F>
void run_case(const std::string& name, F f)
{
    g_case = name;
    int before = g_failures;
    try
    {
        f();
    }
    catch (const std::exception& e)
    {
        printf("FAIL %s: exception %s\n", name.c_str(), e.what());
        ++g_failures;
    }
    if (g_failures == before)
        printf("PASS %s\n", name.c_str());
}

// ---- fake operator and emitters ----------------------------------------------------------------
REGISTER_OP(FakeOp).attr<int>("answer", 42).infershape([](std::shared_ptr<graph::GNode> gnode) -> void {
    gnode->set_output_type_and_shape(0, gnode->get_input_element_type(0), gnode->get_input_shape(0));
});

namespace
{
    std::vector<std::string> g_emit_log;

    class FakeEmitter : public KernelEmitter
    {
    public:
        FakeEmitter(std::shared_ptr<KernelContext> ctx, const std::string& type, const std::string& label, bool declines)
            : KernelEmitter(ctx, type)
            , m_label(label)
            , m_declines(declines)
        {
        }
        LanguageUnit_p emit_function_body() override
        {
            g_emit_log.push_back(m_label);
            if (m_declines)
                return nullptr;
            LanguageUnit_p lu(new LanguageUnit(get_function_name()));
            *lu << "// body of " << m_label << "\n";
            return lu;
        }
        LanguageUnit_p emit_dependency() override
        {
            LanguageUnit_p lu(new LanguageUnit(get_function_name() + "_dep"));
            lu->require(header::stdio);
            return lu;
        }
        std::string m_label;
        bool m_declines;
    };

    struct RocmLow : FakeEmitter { RocmLow(std::shared_ptr<KernelContext> c) : FakeEmitter(c, "rocm", "rocm_p2", false) {} };
    struct RocmHighDeclines : FakeEmitter { RocmHighDeclines(std::shared_ptr<KernelContext> c) : FakeEmitter(c, "rocm", "rocm_p7_declines", true) {} };
    struct CudaMid : FakeEmitter { CudaMid(std::shared_ptr<KernelContext> c) : FakeEmitter(c, "cuda", "cuda_p3", false) {} };
    struct CudaSame : FakeEmitter { CudaSame(std::shared_ptr<KernelContext> c) : FakeEmitter(c, "cuda", "cuda_p2", false) {} };
    struct F16Only : FakeEmitter { F16Only(std::shared_ptr<KernelContext> c) : FakeEmitter(c, "rocm", "rocm_f16_p9", false) {} };
    struct CpuOnly : FakeEmitter { CpuOnly(std::shared_ptr<KernelContext> c) : FakeEmitter(c, "cpu", "cpu_p9", false) {} };
} // namespace

REGISTER_KERNEL_EMITTER("FakeOp", Device(ROCM_GPU).TypeConstraint(element::f32).Tag("low").Priority(2), RocmLow)
REGISTER_KERNEL_EMITTER("FakeOp", Device(ROCM_GPU).TypeConstraint(element::f32).Tag("high").Priority(7), RocmHighDeclines)
REGISTER_KERNEL_EMITTER("FakeOp", Device(CUDA_GPU).TypeConstraint(element::f32).Tag("mid").Priority(3), CudaMid)
REGISTER_KERNEL_EMITTER("FakeOp", Device(CUDA_GPU).TypeConstraint(element::f32).Tag("same").Priority(2), CudaSame)
REGISTER_KERNEL_EMITTER("FakeOp", Device(ROCM_GPU).TypeConstraint(element::f16).Tag("f16").Priority(9), F16Only)
REGISTER_KERNEL_EMITTER("FakeOp", Device(GENERIC_CPU).TypeConstraint(element::f32).Tag("cpu").Priority(9), CpuOnly)

namespace
{
    std::shared_ptr<graph::GNode> param(graph::Graph& g, const element::Type& t, const Shape& s)
    {
        return g.add_node_and_edge(std::make_shared<op::Parameter>(t, s), graph::GNodeVector{});
    }

    std::shared_ptr<graph::GNode> quant_dot_graph(graph::Graph& g, size_t M, size_t N, size_t K, const std::string& cfg = "",
                                                  bool with_gamma = false, bool with_bias = false, bool with_res = false,
                                                  size_t rows_mul = 1)
    {
        auto a = param(g, element::f16, Shape{M, K});
        auto w = param(g, element::u8, Shape{N * rows_mul, K / 2});
        auto s = param(g, element::f16, Shape{N * rows_mul, K / 128});
        graph::GNodeVector in{a, w, s};
        if (with_gamma)
            in.push_back(param(g, element::f16, Shape{K}));
        if (with_bias)
            in.push_back(param(g, element::f16, Shape{N}));
        if (with_res)
            in.push_back(param(g, element::f16, Shape{M, N}));
        auto config = cfg.empty() ? op::OpConfig::any() : op::OpConfig::any::parse(cfg);
        return g.add_node_and_edge(std::make_shared<op::GenericOp>("qd", "QuantDot", config), in);
    }

    std::string read_file(const std::string& path)
    {
        std::ifstream f(path);
        std::stringstream ss;
        ss << f.rdbuf();
        return ss.str();
    }
} // namespace

int main(int argc, char** argv)
{
    const std::string tmp = argc > 1 ? argv[1] : "/tmp/nnf_host_test";
    // where tests/golden lives (second argument; default: relative to the repository root as working directory)
    const std::string golden = argc > 2 ? argv[2] : "tests/golden";

    run_case("element_types", [] {
        EXPECT(element::f16.c_type_string() == "half" && element::f16.size() == 2);
        EXPECT(element::u8.c_type_string() == "uint8_t" && element::u8.is_quantized() && !element::u8.is_signed());
        EXPECT(element::i8.c_type_string() == "int8_t" && element::i8.is_quantized());
        EXPECT(element::f32.c_type_string() == "float" && element::f32.is_real());
        element::Type merged;
        EXPECT(!element::Type::merge(merged, element::f16, element::u8)); // why a quantized Dot cannot be op::Dot
        EXPECT(element::Type::merge(merged, element::f16, element::f16) && merged == element::f16);
        EXPECT(get_device_str(ROCM_GPU) == "ROCM_GPU" && (int)ROCM_GPU == 1 && get_device_type("ROCm") == ROCM_GPU);
    });

    run_case("language_units", [] {
        LanguageUnit_p h(new LanguageUnit("header::a", "#include <a>\n"));
        LanguageUnit_p m(new LanguageUnit("macro::b", "#define B\n"));
        LanguageUnit_p d(new LanguageUnit("declaration::c", "typedef int c;\n"));
        LanguageUnit_p body(new LanguageUnit("body", "body();\n"));
        body->require(d);
        body->require(m);
        body->require(h);
        EXPECT(body->collect_code() == "#include <a>\n#define B\ntypedef int c;\nbody();\n");
        EXPECT(body->required.count("macro::b") == 1);
        body->clean_require();
        EXPECT(body->collect_code() == "body();\n");
        LanguageUnit w("w");
        w << "if (x)\n";
        w.block_begin();
        w << "y();\n";
        w.block_end();
        EXPECT(w.get_code() == "if (x)\n{\n    y();\n}\n");
        FunctionUnit fu;
        fu.name_unit = LanguageUnit_p(new LanguageUnit("n", "my_kernel"));
        fu.signature_unit = LanguageUnit_p(new LanguageUnit("s", "void (float* input0, float* output0)"));
        fu.call_unit = LanguageUnit_p(new LanguageUnit("c", "(a, b);\n"));
        EXPECT(fu.get_specialized_signature() == "void my_kernel(float* input0, float* output0)");
        EXPECT(fu.get_specialized_function_call() == "my_kernel(a, b);\n");
        EXPECT(fu.get_specialized_function_call("other") == "other(a, b);\n");
    });

    run_case("json_lite", [] {
        auto j = json_lite::parse("{\"group\": 128, \"eps\": 1e-6, \"act\": \"silu_gate\", \"flag\": true, \"v\": [1, 2, 3]}");
        EXPECT(j["group"].get<int>() == 128 && j["flag"].get<bool>() && j["act"].get<std::string>() == "silu_gate");
        EXPECT(j["eps"].get<double>() == 1e-6 && j["v"].size() == 3 && j["v"][2].get<int>() == 3);
        EXPECT(json_lite::parse(j.dump()).dump() == j.dump());
        bool threw = false;
        try
        {
            json_lite::parse("{\"a\": }");
        }
        catch (const CheckError&)
        {
            threw = true;
        }
        EXPECT(threw);
    });

    run_case("registry_lookup", [] {
        auto* reg = KernelRegistry::Global();
        EXPECT(reg->FindKernelRegistrations("FakeOp", ROCM_GPU, element::f32).size() == 2);
        EXPECT(reg->FindKernelRegistrations("FakeOp", CUDA_GPU, element::f32).size() == 2);
        EXPECT(reg->FindKernelRegistrations("FakeOp", ROCM_GPU, element::f16).size() == 1);
        EXPECT(reg->FindKernelRegistrations("NoSuchOp", ROCM_GPU, element::f32).empty());
        auto best = reg->FindKernelRegistration("FakeOp", ROCM_GPU, element::f32);
        EXPECT(best && best->m_tag == "high" && best->m_priority == 7);
        // the automatic emitter (priority 5) and four kernel variants (priority 3)
        EXPECT(reg->FindKernelRegistrations("QuantDot", ROCM_GPU, element::f32).size() == 5);
        auto qd = reg->FindKernelRegistration("QuantDot", ROCM_GPU, element::f32);
        EXPECT(qd && qd->m_tag == "nnf_hip_gfx950" && qd->m_priority == 5);
        EXPECT(reg->FindKernelRegistrations("QuantDotW8A8", ROCM_GPU, element::f32).size() == 1);
        EXPECT(reg->FindKernelRegistrations("FusedQuantMLP", ROCM_GPU, element::f32).size() == 1);
        bool threw = false;
        try
        {
            Name("Broken").Device(ROCM_GPU).Build(); // no factory
        }
        catch (const CheckError&)
        {
            threw = true;
        }
        EXPECT(threw);
    });

    run_case("selection_order_and_decline", [] {
        graph::Graph g;
        auto x = param(g, element::f16, Shape{2, 3}); // fp16 node: the lookup key is still element::f32
        auto node = g.add_node_and_edge(std::make_shared<op::GenericOp>("fake", "FakeOp", op::OpConfig::any()), {x});
        pass::graph::DefaultKernelSelector sel;
        g_emit_log.clear();
        auto ans = sel.pick_first(node, ROCM_GPU);
        EXPECT(ans.second != nullptr);
        // candidates: rocm_p7 (7+1, declines), cuda_p3 (3), rocm_p2 (2+1), cuda_p2 (2): tie 3 vs 3 broken by
        // kernel type string "cuda" < "rocm"
        EXPECT(g_emit_log.size() == 2 && g_emit_log[0] == "rocm_p7_declines" && g_emit_log[1] == "cuda_p3");
        auto* won = dynamic_cast<FakeEmitter*>(ans.second.get());
        EXPECT(won && won->m_label == "cuda_p3");
        EXPECT(ans.second->get_device_type() == CUDA_GPU && ans.first == ROCM_GPU);
        // the f16 registration (priority 9) and the CPU one are never candidates for a ROCm node
        for (auto& l : g_emit_log)
            EXPECT(l != "rocm_f16_p9" && l != "cpu_p9");
        // on a CUDA node only CUDA registrations are looked at
        g_emit_log.clear();
        auto ans2 = sel.pick_first(node, CUDA_GPU);
        EXPECT(dynamic_cast<FakeEmitter*>(ans2.second.get())->m_label == "cuda_p3" && g_emit_log.size() == 1);
        // no registration at all
        auto ans3 = sel.pick_first(node, HLSL);
        EXPECT(ans3.second == nullptr);
    });

    run_case("emitter_name_signature_call", [] {
        graph::Graph g;
        auto x = param(g, element::f16, Shape{2, 3});
        auto node = g.add_node_and_edge(std::make_shared<op::GenericOp>("fake", "FakeOp", op::OpConfig::any()), {x});
        auto ctx = std::make_shared<KernelContext>(node);
        EXPECT(ctx->dtypes.size() == 2 && ctx->dtypes[0] == "half" && ctx->gpu_num_sm == 20);
        EXPECT(ctx->generate_identifier() == "FakeOp_i2x3_o2x3_half_half");
        RocmLow k(ctx);
        auto fu = k.get_or_emit_source();
        EXPECT(fu != nullptr && k.is_emitted());
        const std::string uname = node->get_op_ptr()->get_unique_name();
        EXPECT(fu->name_unit->get_code() == "FakeOp_half_half_rocm_" + uname);
        EXPECT(fu->signature_unit->get_code() == "void (half* input0, half* output0)");
        EXPECT(fu->call_unit->get_code() == "(" + x->get_output_tensor_ptr(0)->get_name() + ", " +
                                                node->get_output_tensor_ptr(0)->get_name() + ");\n");
        // body requires dep, call requires body (orders headers before kernels)
        EXPECT(fu->body_unit->required.count(fu->dep_unit->symbol) == 1);
        EXPECT(fu->call_unit->required.count(fu->body_unit->symbol) == 1);
        CONTAINS(fu->comment_unit->get_code(), "// Description:\tFakeOp");
        // second call returns the same unit; with emit_func_call the call unit is rebuilt
        auto before = fu->call_unit;
        EXPECT(k.get_or_emit_source() == fu && fu->call_unit == before);
        EXPECT(k.get_or_emit_source(true) == fu && fu->call_unit != before);
        RocmHighDeclines d(ctx);
        EXPECT(d.get_or_emit_source() == nullptr);
    });

    run_case("quant_dot_infershape", [] {
        graph::Graph g;
        auto n = quant_dot_graph(g, 1, 4096, 4096);
        EXPECT(n->get_output_shape(0) == (Shape{1, 4096}) && n->get_output_element_type(0) == element::f16);
        graph::Graph g2;
        auto n2 = quant_dot_graph(g2, 256, 11008, 4096, "{\"act\": \"silu_gate\", \"rms_norm\": true}", true, false, false, 2);
        EXPECT(n2->get_output_shape(0) == (Shape{256, 11008}));
        // wrong scale shape, wrong packing, wrong input count, bad attribute
        auto expect_throw = [](std::function<void()> f) {
            bool threw = false;
            try
            {
                f();
            }
            catch (const CheckError&)
            {
                threw = true;
            }
            return threw;
        };
        EXPECT(expect_throw([] {
            graph::Graph g3;
            auto a = param(g3, element::f16, Shape{1, 256});
            auto w = param(g3, element::u8, Shape{8, 128});
            auto s = param(g3, element::f16, Shape{8, 1}); // K/group = 2 expected
            g3.add_node_and_edge(std::make_shared<op::GenericOp>("x", "QuantDot", op::OpConfig::any()), {a, w, s});
        }));
        EXPECT(expect_throw([] {
            graph::Graph g3;
            auto a = param(g3, element::f16, Shape{1, 256});
            auto w = param(g3, element::u8, Shape{8, 256}); // not K/2
            auto s = param(g3, element::f16, Shape{8, 2});
            g3.add_node_and_edge(std::make_shared<op::GenericOp>("x", "QuantDot", op::OpConfig::any()), {a, w, s});
        }));
        EXPECT(expect_throw([] {
            graph::Graph g3;
            quant_dot_graph(g3, 1, 8, 256, "{\"has_bias\": true}"); // bias input missing
        }));
        EXPECT(expect_throw([] {
            graph::Graph g3;
            quant_dot_graph(g3, 1, 8, 256, "{\"zero_point\": 16}");
        }));
        EXPECT(expect_throw([] {
            graph::Graph g3;
            quant_dot_graph(g3, 1, 8, 256, "{\"act\": \"gelu\"}");
        }));
    });

    run_case("quant_dot_emitter_text", [] {
        graph::Graph g;
        auto n = quant_dot_graph(g, 1, 12288, 4096);
        pass::graph::DefaultKernelSelector sel;
        auto ans = sel.pick_first(n, ROCM_GPU);
        EXPECT(ans.second != nullptr && ans.second->get_kernel_type() == "rocm");
        auto fu = ans.second->get_or_emit_source();
        EXPECT(fu->name_unit->get_code() == "QuantDot_half_uint8_t_half_half_rocm_" + n->get_op_ptr()->get_unique_name());
        EXPECT(fu->signature_unit->get_code() == "void (hipStream_t stream, half* input0, uint8_t* input1, half* input2, half* output0)");
        EXPECT(fu->body_unit->get_code() ==
               "NNF_HIP_CHECK(nnf_w4a16_gemm(stream, input0, input1, input2, output0, 1, 12288, 4096, 128, 8, nullptr, 0));\n");
        // the signature asks for a stream, so the call starts with one
        CONTAINS(fu->call_unit->get_code(), "(0, ");
        std::string deps = fu->dep_unit->collect_required_code();
        CONTAINS(deps, "#include <hip/hip_runtime.h>");
        CONTAINS(deps, "#include \"nnf_hip_kernels.h\"");
        CONTAINS(deps, "#define NNF_HIP_CHECK(x)");
        CONTAINS(deps, "typedef _Float16 half;");
        EXPECT(deps.find("cuda") == std::string::npos && deps.find("cublas") == std::string::npos);

        // fused variant: gamma, bias; the scratch tensor appears in signature and call.  Its size: one fp32 per row
        // (rstd) + the parked sums of the plan for this shape (64 tiles of 128 x 128 -- 256-row tiles would leave 32 -- x 16 supersteps
        // over 256 workgroups: one slot each)
        graph::Graph g2;
        auto n2 = quant_dot_graph(g2, 256, 4096, 4096, "{\"rms_norm\": true, \"has_bias\": true, \"rms_eps\": 1e-5}", true, true);
        auto k2 = sel.pick_first(n2, ROCM_GPU).second;
        auto fu2 = k2->get_or_emit_source();
        CONTAINS(fu2->body_unit->get_code(), "nnf_w4a16_gemm_fused_variant(stream, input0, input1, input2, output0, 256, 4096, 4096, 128, 8, input3, 1.000000000e-05f, input4, nullptr, NNF_ACT_NONE, NNF_W4A16_AUTO, &plan, ");
        // ... and, because the product runs on the tile GEMM, a second tensor: its synchronisation words (two for rstd[],
        // two per tile: 2 x 32 tiles; in whole 64 bytes), persistent and cleared at initialisation, named by the nnf_plan
        // the body declares
        EXPECT(k2->m_context->tensors.size() == 2 &&
               k2->m_context->tensors[0]->size() == (size_t)256 * 4 + (size_t)256 * 128 * 128 * 4);
        EXPECT(k2->m_context->tensors[1]->size() == 576 && k2->m_context->tensors[1]->is_persistent() &&
               k2->m_context->tensors[1]->is_memset() && k2->m_context->tensors[1]->get_memset_value() == 0);
        CONTAINS(fu2->body_unit->get_code(), "const nnf_plan plan = {0, 0, 0, " + k2->m_context->tensors[1]->get_name() + ", 576, 0};");
        CONTAINS(fu2->signature_unit->get_code(), "char* " + k2->m_context->tensors[0]->get_name());
        CONTAINS(fu2->call_unit->get_code(), k2->m_context->tensors[1]->get_name() + ");");
        // SiLU gate: N is half the weight rows
        graph::Graph g3;
        auto n3 = quant_dot_graph(g3, 256, 11008, 4096, "{\"act\": \"silu_gate\"}", false, false, false, 2);
        CONTAINS(sel.pick_first(n3, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                 "256, 11008, 4096, 128, 8, nullptr, 1.000000000e-06f, nullptr, nullptr, NNF_ACT_SILU_GATE");
    });

    run_case("quant_dot_emitter_declines", [] {
        pass::graph::DefaultKernelSelector sel;
        {
            graph::Graph g; // groups of 16 are a legal op, but no kernel serves them
            auto a = param(g, element::f16, Shape{1, 256});
            auto w = param(g, element::u8, Shape{8, 128});
            auto s = param(g, element::f16, Shape{8, 16});
            auto n = g.add_node_and_edge(std::make_shared<op::GenericOp>("x", "QuantDot", op::OpConfig::any::parse("{\"group_size\": 16}")),
                                         {a, w, s});
            EXPECT(sel.pick_first(n, ROCM_GPU).second == nullptr);
        }
        {
            graph::Graph g; // fp32 activations
            auto a = param(g, element::f32, Shape{1, 256});
            auto w = param(g, element::u8, Shape{8, 128});
            auto s = param(g, element::f16, Shape{8, 2});
            auto n = g.add_node_and_edge(std::make_shared<op::GenericOp>("x", "QuantDot", op::OpConfig::any()), {a, w, s});
            EXPECT(sel.pick_first(n, ROCM_GPU).second == nullptr);
        }
        {
            graph::Graph g; // gate + bias has no fused kernel
            auto n = quant_dot_graph(g, 4, 8, 256, "{\"act\": \"silu_gate\", \"has_bias\": true}", false, true, false, 2);
            EXPECT(sel.pick_first(n, ROCM_GPU).second == nullptr);
        }
        {
            graph::Graph g; // a CUDA node finds no emitter for this op
            auto n = quant_dot_graph(g, 1, 8, 256);
            EXPECT(sel.pick_first(n, CUDA_GPU).second == nullptr);
        }
    });

    run_case("w8a8_and_mlp_emitters", [] {
        pass::graph::DefaultKernelSelector sel;
        graph::Graph g;
        auto a = param(g, element::i8, Shape{32, 8192});
        auto st = param(g, element::f32, Shape{32});
        auto w = param(g, element::i8, Shape{8192, 8192});
        auto sc = param(g, element::f32, Shape{8192});
        auto n = g.add_node_and_edge(std::make_shared<op::GenericOp>("q", "QuantDotW8A8", op::OpConfig::any()), {a, st, w, sc});
        EXPECT(n->get_output_element_type(0) == element::f16 && n->get_output_shape(0) == (Shape{32, 8192}));
        auto kq = sel.pick_first(n, ROCM_GPU).second;
        auto fu = kq->get_or_emit_source();
        // M = 32: 64 x 256 tiles (32 of them), K split 8 ways: 8 x 32 x 8192 int32 partial sums in a scratch tensor; the
        // row-streaming kernel, which the library prefers here, runs over two ranges of K that meet at a word per workgroup
        EXPECT(kq->m_context->tensors.size() == 2 && kq->m_context->tensors[0]->size() == (size_t)8 * 32 * 8192 * 4 &&
               kq->m_context->tensors[1]->size() == 1024 && kq->m_context->tensors[1]->is_persistent());
        EXPECT(fu->body_unit->get_code() ==
               "const nnf_plan plan = {0, 0, 0, " + kq->m_context->tensors[1]->get_name() + ", 1024, 0};\n" +
                   "NNF_HIP_CHECK(nnf_w8a8_gemm_variant(stream, input0, input1, input2, input3, output0, nullptr, 32, 8192, 8192, "
                   "NNF_W8A8_AUTO, &plan, " +
                   kq->m_context->tensors[0]->get_name() + ", 8388608));\n");
        auto n2 = g.add_node_and_edge(std::make_shared<op::GenericOp>("q", "QuantDotW8A8", op::OpConfig::any::parse("{\"out_type\": \"i32\"}")),
                                      {a, st, w, sc});
        EXPECT(n2->get_output_element_type(0) == element::i32);
        CONTAINS(sel.pick_first(n2, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                 "nnf_w8a8_gemm_variant(stream, input0, nullptr, input2, nullptr, nullptr, output0, 32, 8192, 8192, NNF_W8A8_AUTO, &plan, ");
        {
            // a product the tile GEMM takes: the plain calls
            graph::Graph g3;
            auto a3 = param(g3, element::i8, Shape{512, 8192});
            auto st3 = param(g3, element::f32, Shape{512});
            auto n3 = g3.add_node_and_edge(std::make_shared<op::GenericOp>("q", "QuantDotW8A8", op::OpConfig::any()),
                                           {a3, st3, param(g3, element::i8, Shape{8192, 8192}), param(g3, element::f32, Shape{8192})});
            CONTAINS(sel.pick_first(n3, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                     "nnf_w8a8_gemm(stream, input0, input1, input2, input3, output0, 512, 8192, 8192");
            auto n4 = g3.add_node_and_edge(std::make_shared<op::GenericOp>("q", "QuantDotW8A8", op::OpConfig::any::parse("{\"out_type\": \"i32\"}")),
                                           {a3, st3, param(g3, element::i8, Shape{8192, 8192}), param(g3, element::f32, Shape{8192})});
            CONTAINS(sel.pick_first(n4, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                     "nnf_w8a8_gemm_acc(stream, input0, input2, output0, 512, 8192, 8192");
        }

        graph::Graph g2;
        auto x = param(g2, element::f16, Shape{256, 4096});
        auto gamma = param(g2, element::f16, Shape{4096});
        auto wgu = param(g2, element::u8, Shape{22016, 2048});
        auto sgu = param(g2, element::f16, Shape{22016, 32});
        auto wd = param(g2, element::u8, Shape{4096, 5504});
        auto sd = param(g2, element::f16, Shape{4096, 86});
        auto mlp = g2.add_node_and_edge(std::make_shared<op::GenericOp>("mlp", "FusedQuantMLP", op::OpConfig::any()),
                                        {x, gamma, wgu, sgu, wd, sd});
        EXPECT(mlp->get_output_shape(0) == (Shape{256, 4096}));
        auto k = sel.pick_first(mlp, ROCM_GPU).second;
        auto fm = k->get_or_emit_source();
        CONTAINS(fm->body_unit->get_code(), "nnf_fused_mlp_w4a16_planned(stream, input0, input1, 1.000000000e-06f, input2, input3, input4, input5, output0, 256, 4096, 11008, 128, 8, &gate_up_plan, &down_plan, ");
        // rstd [256] fp32 + h [256, 11008] fp16 + the larger of the two areas of parked sums: gate/up (2 x 86 tiles of
        // 128 x 256 weight rows, two thirds of the CUs) runs whole tiles, one workgroup each, and parks nothing; down
        // (2 x 32 tiles of 128 x 128, 43 supersteps each, split evenly over 256 workgroups) one slot per workgroup
        // ... and the synchronisation words of either product (2 x 86 and 2 x 32 tiles, two words each, and two more)
        EXPECT(k->m_context->tensors.size() == 3 &&
               k->m_context->tensors[0]->size() ==
                   (size_t)256 * 4 + (size_t)256 * 11008 * 2 + (size_t)256 * 128 * 128 * 4);
        EXPECT(k->m_context->tensors[1]->size() == 1408 && k->m_context->tensors[2]->size() == 576 &&
               k->m_context->tensors[1]->is_memset() && k->m_context->tensors[2]->is_memset());
    });

    run_case("codegen_project", [&] {
        auto g = std::make_shared<graph::Graph>();
        auto a = param(*g, element::f16, Shape{4, 256});
        std::vector<uint8_t> wbytes(16 * 128, 0x98);
        std::vector<uint16_t> sbytes(16 * 2, 0x2000);
        auto w = g->add_node_and_edge(std::make_shared<op::Constant>(element::u8, Shape{16, 128}, wbytes.data()), graph::GNodeVector{});
        auto s = g->add_node_and_edge(std::make_shared<op::Constant>(element::f16, Shape{16, 2}, sbytes.data()), graph::GNodeVector{});
        // two layers with identical shapes share one definition; a third with another N gets its own
        auto l1 = g->add_node_and_edge(std::make_shared<op::GenericOp>("l1", "QuantDot", op::OpConfig::any()), {a, w, s});
        auto l2 = g->add_node_and_edge(std::make_shared<op::GenericOp>("l2", "QuantDot", op::OpConfig::any()), {a, w, s});
        std::vector<uint8_t> w2bytes(32 * 128, 0x77);
        std::vector<uint16_t> s2bytes(32 * 2, 0x2000);
        auto w2 = g->add_node_and_edge(std::make_shared<op::Constant>(element::u8, Shape{32, 128}, w2bytes.data()), graph::GNodeVector{});
        auto s2 = g->add_node_and_edge(std::make_shared<op::Constant>(element::f16, Shape{32, 2}, s2bytes.data()), graph::GNodeVector{});
        auto l3 = g->add_node_and_edge(std::make_shared<op::GenericOp>("l3", "QuantDot", op::OpConfig::any()), {a, w2, s2});
        auto r1 = g->add_node_and_edge(std::make_shared<op::Result>(), {l1});
        auto r2 = g->add_node_and_edge(std::make_shared<op::Result>(), {l2});
        auto r3 = g->add_node_and_edge(std::make_shared<op::Result>(), {l3});
        (void)r1; (void)r2; (void)r3;

        ROCmEngine engine(tmp + "/codegen_project/");
        engine.pass.exit_after_codegen = false;
        engine.pass.kernels_include_dir = "/inc";
        engine.pass.kernels_lib_dir = "/lib";
        EXPECT(engine.run_on_graph(g));
        auto& trace = engine.pass.hook_trace;
        std::vector<std::string> expected{"initialize", "collect_mem", "collect_stream", "collect_funcs", "modify_codegen", "codegen", "after_projgen"};
        EXPECT(trace == expected);
        EXPECT((*l1)["Kernel_Selection_Result"].is_valid() && (*l1)["DeviceType"].as<NNFusion_DeviceType>() == ROCM_GPU);

        std::string rt = read_file(tmp + "/codegen_project/nnfusion_rt.cpp");
        std::string hdr = read_file(tmp + "/codegen_project/nnfusion_rt.h");
        std::string mk = read_file(tmp + "/codegen_project/Makefile");
        std::string pj = read_file(tmp + "/codegen_project/para_info.json");
        std::string mt = read_file(tmp + "/codegen_project/main_test.cpp");
        EXPECT(!rt.empty() && !hdr.empty() && !mk.empty() && !pj.empty() && !mt.empty());
        // headers before macros before declarations before code
        size_t p_h = rt.find("#include <hip/hip_runtime.h>"), p_m = rt.find("#define NNF_HIP_CHECK"), p_d = rt.find("typedef _Float16 half;"),
               p_k = rt.find("void QuantDot_half_uint8_t_half_half_rocm_");
        EXPECT(p_h != std::string::npos && p_h < p_m && p_m < p_d && p_d < p_k);
        // l1 and l2: one definition, two calls; l3: its own definition
        size_t defs = 0, pos = 0;
        while ((pos = rt.find("\nvoid QuantDot_half_uint8_t_half_half_rocm_", pos)) != std::string::npos)
        {
            ++defs;
            ++pos;
        }
        EXPECT(defs == 2);
        const std::string f1 = "QuantDot_half_uint8_t_half_half_rocm_" + l1->get_op_ptr()->get_unique_name();
        size_t calls = 0;
        pos = 0;
        while ((pos = rt.find(f1 + "(nnf_stream_0, ", pos)) != std::string::npos)
        {
            ++calls;
            ++pos;
        }
        EXPECT(calls == 2);
        CONTAINS(rt, "extern \"C\" int kernel_entry(half* " + a->get_output_tensor_ptr(0)->get_name());
        CONTAINS(rt, "extern \"C\" void rocm_init()");
        CONTAINS(rt, "extern \"C\" void cuda_init()");
        CONTAINS(rt, "extern \"C\" int get_device_type()\n{\n    return 1;");
        CONTAINS(rt, "nnf_load_constant((void**)&" + w->get_output_tensor_ptr(0)->get_name() + ", \"./Constant/" +
                         w->get_output_tensor_ptr(0)->get_name() + ".bin\", 2048);");
        CONTAINS(rt, "nnf_w4a16_gemm(stream, input0, input1, input2, output0, 4, 16, 256, 128, 8, nullptr, 0)");
        CONTAINS(rt, "nnf_w4a16_gemm(stream, input0, input1, input2, output0, 4, 32, 256, 128, 8, nullptr, 0)");
        // results are written in place: the producing tensor aliases the caller's buffer
        CONTAINS(rt, "half* " + l1->get_output_tensor_ptr(0)->get_name() + " = " + r1->get_output_tensor_ptr(0)->get_name() + ";");
        // HIP text only
        for (const char* banned : {"cuda_runtime", "cublas", "cudnn", "hipify", "rocm_adapter", "__global__"})
            EXPECT(rt.find(banned) == std::string::npos);
        CONTAINS(hdr, "extern \"C\" int64_t get_workspace_size();");
        CONTAINS(mk, "--offload-arch=gfx950");
        CONTAINS(mk, "NNF_INC ?= /inc");
        CONTAINS(pj, "\"shape\": [4, 256]");
        CONTAINS(mt, "Summary: [min, max, mean]");
        std::string cbin = read_file(tmp + "/codegen_project/Constant/" + w->get_output_tensor_ptr(0)->get_name() + ".bin");
        EXPECT(cbin.size() == 2048 && (uint8_t)cbin[0] == 0x98);
    });

    run_case("profiler_harness_source", [&] {
        graph::Graph g;
        auto n = quant_dot_graph(g, 2, 64, 256);
        pass::graph::DefaultKernelSelector sel;
        auto k = sel.pick_first(n, ROCM_GPU).second;
        auto pc = std::make_shared<profiler::ProfilingContext>(k);
        pc->warmup_times = 2;
        pc->runtime_times = 7;
        profiler::HipDefaultRuntime rt("/inc", "/lib");
        EXPECT(rt.codegen(pc));
        EXPECT(pc->entry_name == k->get_function_name() + "_entry");
        CONTAINS(pc->source_code, "extern \"C\" double " + pc->entry_name + "(void** args, void** outputs)");
        CONTAINS(pc->source_code, "(half*)args[0], (uint8_t*)args[1], (half*)args[2], (half*)outputs[0]");
        CONTAINS(pc->source_code, "for (size_t i = 0; i < 7; ++i)");
        CONTAINS(pc->source_code, "return (double)ms / 7;");
        CONTAINS(pc->source_code, "hipMemcpyHostToDevice");
    });

    run_case("profiling_selector_candidates", [&] {
        // the automatic emitter and the kernel variants that can serve the shape, in priority order; the
        // default selector keeps picking the automatic one
        auto kinds = [](size_t M, size_t N, size_t K, const std::string& cfg = "", bool gamma = false) {
            graph::Graph g;
            auto n = quant_dot_graph(g, M, N, K, cfg, gamma);
            pass::graph::ProfilingBasedKernelSelector sel;
            std::vector<std::string> out;
            for (auto& k : sel.candidates(n, ROCM_GPU))
                out.push_back(k->get_kernel_type());
            pass::graph::DefaultKernelSelector def;
            EXPECT(def.pick_first(n, ROCM_GPU).second->get_kernel_type() == "rocm");
            return out;
        };
        auto has = [](const std::vector<std::string>& v, const std::string& x) {
            return std::find(v.begin(), v.end(), x) != v.end();
        };
        auto k1 = kinds(1, 4096, 4096);
        EXPECT(k1.size() == 5 && k1[0] == "rocm");
        EXPECT(has(k1, "rocm_gemv_rows") && has(k1, "rocm_gemv_mfma") && has(k1, "rocm_gemm_mfma") && has(k1, "rocm_gemv_valu"));
        auto k8 = kinds(8, 4096, 4096);
        EXPECT(k8.size() == 5 && has(k8, "rocm_gemv_rows")); // 2 .. 16 rows: the row-streaming MFMA kernel
        auto k8odd = kinds(8, 4096, 4224);                   // ... which takes multiples of 256 (1024 .. 8192) only
        EXPECT(k8odd.size() == 4 && !has(k8odd, "rocm_gemv_rows"));
        auto k16 = kinds(16, 8192, 8192); // too many activations for one workgroup's LDS: the MFMA GEMV over ranges of K
        EXPECT(has(k16, "rocm_gemv_mfma") && has(k16, "rocm_gemm_mfma"));
        auto k40 = kinds(40, 8192, 8192); // more rows than any GEMV kernel takes
        EXPECT(k40.size() == 2 && !has(k40, "rocm_gemv_mfma") && !has(k40, "rocm_gemv_rows"));
        auto kbig = kinds(4096, 8192, 8192);
        EXPECT(kbig.size() == 2 && kbig[1] == "rocm_gemm_mfma");
        auto kfused = kinds(4, 256, 256, "{\"rms_norm\": true}", true);
        EXPECT(kfused.size() == 1 && kfused[0] == "rocm");
        // the emitted call names the variant; the harness source of a variant differs from the automatic one's
        graph::Graph g;
        auto n = quant_dot_graph(g, 1, 4096, 4096);
        pass::graph::ProfilingBasedKernelSelector sel;
        sel.runtime_times = 9;
        profiler::HipDefaultRuntime rt("/inc", "/lib");
        auto pcs = sel.contexts(n, ROCM_GPU, rt);
        EXPECT(pcs.size() == 5);
        size_t rows = 0;
        for (auto& pc : pcs)
        {
            CONTAINS(pc->source_code, "for (size_t i = 0; i < 9; ++i)");
            if (pc->kernel->get_kernel_type() == "rocm_gemv_rows")
            {
                ++rows;
                CONTAINS(pc->source_code, "nnf_w4a16_gemm_variant(stream, input0, input1, input2, output0, 1, 4096, 4096, 128, 8, NNF_W4A16_GEMV_ROWS, nullptr, nullptr, 0)");
                CONTAINS(pc->entry_name, "_rocm_gemv_rows_");
            }
        }
        EXPECT(rows == 1);
        // a disabled selector leaves the graph alone
        auto gp = std::make_shared<graph::Graph>();
        auto n2 = quant_dot_graph(*gp, 1, 4096, 4096);
        pass::graph::DefaultGNodeDeviceDispatcher().run_on_graph(gp);
        sel.enable = false;
        EXPECT(sel.run_on_graph(gp, rt) && !(*n2)["Kernel_Selection_Result"].is_valid());
    });

    run_case("onnx_reader_on_reference_models", [&] {
        using namespace frontend::onnx_lite;
        const std::string dir = golden + "/onnx/";
        // add_abc_initializers: packed int64_data initializer, tensor attribute with packed float_data
        Model m = parse_model_file(dir + "add_abc_initializers.onnx");
        EXPECT(m.ir_version == 3 && m.producer_name == "ngraph ONNXImporter" && m.graph_name == "test_graph");
        EXPECT(m.opset.at("") == 4);
        EXPECT(m.nodes.size() == 3 && m.nodes[0].op_type == "Constant" && m.nodes[1].op_type == "Add" && m.nodes[2].op_type == "Add");
        EXPECT(m.nodes[1].inputs == (std::vector<std::string>{"A", "B"}) && m.nodes[1].outputs == (std::vector<std::string>{"X"}));
        EXPECT(m.nodes[2].inputs == (std::vector<std::string>{"X", "C"}) && m.nodes[2].name == "add_node2");
        const Attribute& val = m.nodes[0].attributes.at("value");
        EXPECT(val.type == 4 && val.t.data_type == FLOAT && val.t.dims == (std::vector<int64_t>{2, 2}) && val.t.name == "const_tensor");
        EXPECT(val.t.bytes.size() == 16);
        float fb[4];
        memcpy(fb, val.t.bytes.data(), 16);
        EXPECT(fb[0] == 1.f && fb[1] == 2.f && fb[2] == 3.f && fb[3] == 4.f);
        EXPECT(m.initializers.size() == 1 && m.initializers[0].name == "A" && m.initializers[0].data_type == INT64);
        int64_t ia[4];
        EXPECT(m.initializers[0].bytes.size() == 32);
        memcpy(ia, m.initializers[0].bytes.data(), 32);
        // the reference's expectation: C = {1,2,3,4} gives Y = A + B + C = {3,6,9,12}
        const float c_in[4] = {1, 2, 3, 4}, want[4] = {3, 6, 9, 12};
        for (int i = 0; i < 4; ++i)
            EXPECT((float)ia[i] + fb[i] + c_in[i] == want[i]);
        EXPECT(m.inputs.size() == 2 && m.inputs[0].name == "A" && m.inputs[1].name == "C" && m.inputs[1].elem_type == FLOAT);
        EXPECT(m.inputs[1].dims == (std::vector<int64_t>{2, 2}) && m.outputs.size() == 1 && m.outputs[0].name == "Y");

        // gemm_op: float and integer attributes, value infos
        Model gm = parse_model_file(dir + "gemm_op.onnx");
        EXPECT(gm.ir_version == 6 && gm.opset.at("") == 11 && gm.graph_name == "gemm" && gm.nodes.size() == 1);
        const Node& ge = gm.nodes[0];
        EXPECT(ge.op_type == "Gemm" && ge.inputs == (std::vector<std::string>{"a", "b", "c"}) && ge.outputs[0] == "y");
        EXPECT(ge.get_float("alpha", 1.f) == 0.25f && ge.get_float("beta", 1.f) == 0.35f);
        EXPECT(ge.get_int("transA", 0) == 1 && ge.get_int("transB", 0) == 1 && ge.get_int("absent", 7) == 7);
        EXPECT(ge.attributes.at("alpha").type == 1 && ge.attributes.at("transA").type == 2);
        EXPECT(gm.inputs.size() == 3 && gm.inputs[0].dims == (std::vector<int64_t>{4, 3}) && gm.inputs[1].dims == (std::vector<int64_t>{5, 4}));
        EXPECT(gm.inputs[2].dims == (std::vector<int64_t>{1, 5}) && gm.outputs[0].dims == (std::vector<int64_t>{3, 5}));

        Model mm = parse_model_file(dir + "matmul_op_3.onnx");
        EXPECT(mm.nodes.size() == 1 && mm.nodes[0].op_type == "MatMul");
        EXPECT(mm.inputs[0].dims == (std::vector<int64_t>{2}) && mm.inputs[1].dims == (std::vector<int64_t>{3, 2, 1}));
        EXPECT(mm.outputs[0].dims == (std::vector<int64_t>{3, 1}));

        // truncated files raise instead of reading past the end
        std::ifstream f(dir + "gemm_op.onnx", std::ios::binary);
        std::vector<uint8_t> bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
        bytes.resize(bytes.size() - 7);
        bool threw = false;
        try
        {
            parse_model(bytes);
        }
        catch (const CheckError&)
        {
            threw = true;
        }
        EXPECT(threw);
        // operators outside the quantized path are refused by the importer, as unsupported operators are in the reference
        threw = false;
        try
        {
            frontend::load_onnx_model(dir + "gemm_op.onnx");
        }
        catch (const CheckError& e)
        {
            threw = std::string(e.what()).find("unsupported operator Gemm") != std::string::npos;
        }
        EXPECT(threw);
        // Add is on the path: the reference's model imports (int64 initializer + float constant: types are the graph's business)
        auto g = frontend::load_onnx_model(dir + "add_abc_initializers.onnx");
        size_t adds = 0, consts = 0, params = 0, results = 0;
        for (auto& n : g->get_nodes())
        {
            adds += n->get_op_type() == "Add";
            consts += n->is_constant();
            params += n->is_parameter();
            results += n->is_output();
        }
        EXPECT(adds == 2 && consts == 2 && params == 1 && results == 1);
        // ... but an Add that no quantized product absorbs has no kernel on this device: code generation stops before
        // writing anything, naming every such node
        threw = false;
        try
        {
            ROCmEngine engine(tmp + "/unfused_project/");
            engine.run_on_graph(g);
        }
        catch (const CheckError& e)
        {
            const std::string what = e.what();
            threw = what.find("no ROCM_GPU kernel for: ") != std::string::npos && what.find("(Add)") != std::string::npos &&
                    what.find("fusion passes did not absorb") != std::string::npos;
            size_t named = 0;
            for (size_t at = what.find("(Add)"); at != std::string::npos; at = what.find("(Add)", at + 1))
                ++named;
            EXPECT(named == 2);
        }
        EXPECT(threw);
        EXPECT(!std::ifstream(tmp + "/unfused_project/nnfusion_rt.hip").good());
    });

    run_case("quant_fusion_passes", [] {
        auto cst = [](graph::Graph& g, const element::Type& t, const Shape& s, uint8_t fill) {
            std::vector<uint8_t> d(shape_size(s) * t.size(), fill);
            return g.add_node_and_edge(std::make_shared<op::Constant>(t, s, d.data()), graph::GNodeVector{});
        };
        auto gen = [](graph::Graph& g, const std::string& name, const std::string& type, const graph::GNodeVector& in,
                      const std::string& cfg = "") {
            return g.add_node_and_edge(
                std::make_shared<op::GenericOp>(name, type, cfg.empty() ? op::OpConfig::any() : op::OpConfig::any::parse(cfg)), in);
        };
        auto count = [](const std::shared_ptr<graph::Graph>& g, const std::string& type) {
            size_t n = 0;
            for (auto& node : g->get_ordered_ops())
                n += node->get_op_type() == type;
            return n;
        };
        auto find = [](const std::shared_ptr<graph::Graph>& g, const std::string& type) {
            for (auto& node : g->get_ordered_ops())
                if (node->get_op_type() == type)
                    return node;
            return std::shared_ptr<graph::GNode>();
        };
        const size_t M = 8, H = 256, I = 384;
        // the unfused MLP block; `extra_gate_user` adds a second Result on the gate projection
        auto build_mlp = [&](bool swish_as_one_node, bool extra_gate_user) {
            auto g = std::make_shared<graph::Graph>();
            auto x = param(*g, element::f16, Shape{M, H});
            auto gamma = cst(*g, element::f16, Shape{H}, 0x3c);
            auto wg = cst(*g, element::u8, Shape{I, H / 2}, 0x11), sg = cst(*g, element::f16, Shape{I, H / 128}, 0x21);
            auto wu = cst(*g, element::u8, Shape{I, H / 2}, 0x12), su = cst(*g, element::f16, Shape{I, H / 128}, 0x22);
            auto wd = cst(*g, element::u8, Shape{H, I / 2}, 0x13), sd = cst(*g, element::f16, Shape{H, I / 128}, 0x23);
            auto n = gen(*g, "norm", "RMSNorm", {x, gamma}, "{\"eps\": 1e-5}");
            auto gate = gen(*g, "gate", "QuantDot", {n, wg, sg});
            auto up = gen(*g, "up", "QuantDot", {n, wu, su});
            std::shared_ptr<graph::GNode> act;
            if (swish_as_one_node)
                act = gen(*g, "act", "Swish", {gate});
            else
                act = gen(*g, "act", "Multiply", {gen(*g, "sig", "Sigmoid", {gate}), gate});
            auto h = gen(*g, "h", "Multiply", {up, act});
            auto down = gen(*g, "down", "QuantDot", {h, wd, sd});
            auto out = gen(*g, "out", "Add", {down, x});
            g->add_node_and_edge(std::make_shared<op::Result>(), {out});
            if (extra_gate_user)
                g->add_node_and_edge(std::make_shared<op::Result>(), {gate});
            return g;
        };
        for (int variant = 0; variant < 2; ++variant)
        {
            auto g = build_mlp(variant == 0, false);
            pass::graph::QuantEpilogueFusionPass fusion;
            EXPECT(fusion.run_on_graph(g));
            // everything folds into one node: parameter, gamma, 4 stacked/kept constants, the MLP, the result
            EXPECT(count(g, "FusedQuantMLP") == 1 && count(g, "QuantDot") == 0 && count(g, "RMSNorm") == 0 &&
                   count(g, "Multiply") == 0 && count(g, "Add") == 0 && count(g, "Swish") == 0 && count(g, "Sigmoid") == 0);
            EXPECT(g->get_ordered_ops().size() == 8);
            auto mlp = find(g, "FusedQuantMLP");
            EXPECT(mlp && mlp->get_input_size() == 6 && mlp->get_output_shape(0) == (Shape{M, H}));
            EXPECT(mlp->get_input_shape(2) == (Shape{2 * I, H / 2}) && mlp->get_input_shape(3) == (Shape{2 * I, H / 128}));
            auto wgu = std::dynamic_pointer_cast<op::Constant>(mlp->get_in_edge(2).src->get_op_ptr());
            // gate rows first, then up rows
            EXPECT(wgu && wgu->get_data().front() == 0x11 && wgu->get_data().back() == 0x12 &&
                   wgu->get_data()[I * H / 2 - 1] == 0x11 && wgu->get_data()[I * H / 2] == 0x12);
            auto gop = std::dynamic_pointer_cast<op::GenericOp>(mlp->get_op_ptr());
            EXPECT(std::abs(gop->localOpConfig.getRoot()["rms_eps"].get<double>() - 1e-5) < 1e-12);
            EXPECT(mlp->get_in_edge(0).src->is_parameter() && mlp->get_in_edge(4).src->get_output_shape(0) == (Shape{H, I / 2}));
        }
        {
            // the gate projection is also a graph output: gate and up stay separate; RMSNorm and the residual still fold
            auto g = build_mlp(true, true);
            pass::graph::QuantEpilogueFusionPass fusion;
            EXPECT(fusion.run_on_graph(g));
            EXPECT(count(g, "FusedQuantMLP") == 0 && count(g, "QuantDot") == 3 && count(g, "RMSNorm") == 0 &&
                   count(g, "Add") == 0 && count(g, "Swish") == 1 && count(g, "Multiply") == 1);
            size_t with_rms = 0, with_res = 0;
            for (auto& node : g->get_ordered_ops())
                if (node->get_op_type() == "QuantDot")
                {
                    auto& cfg = std::dynamic_pointer_cast<op::GenericOp>(node->get_op_ptr())->localOpConfig.getRoot();
                    with_rms += cfg["rms_norm"].get<bool>();
                    with_res += cfg["has_residual"].get<bool>();
                }
            EXPECT(with_rms == 2 && with_res == 1);
            // ... and every node that stayed has an emitter of its own: the graph compiles
            pass::graph::DefaultKernelSelector sel;
            for (auto& node : g->get_ordered_ops())
            {
                if (node->is_parameter() || node->is_constant() || node->is_output())
                    continue;
                auto k = sel.pick_first(node, ROCM_GPU).second;
                EXPECT(k != nullptr && k->get_or_emit_source() != nullptr);
            }
            CONTAINS(sel.pick_first(find(g, "Swish"), ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                     "nnf_elementwise_f16(stream, NNF_EW_SWISH, input0, nullptr, output0, 8, 384, 0)");
            CONTAINS(sel.pick_first(find(g, "Multiply"), ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                     "nnf_elementwise_f16(stream, NNF_EW_MULTIPLY, input0, input1, output0, 8, 384, 0)");
        }
        {
            // the nodes around a product as nodes of their own: RMSNorm, Sigmoid, Add with a row operand first
            auto g = std::make_shared<graph::Graph>();
            auto x = param(*g, element::f16, Shape{M, H});
            auto gamma = cst(*g, element::f16, Shape{H}, 0x3c);
            auto row = cst(*g, element::f16, Shape{H}, 0x3c);
            auto n = gen(*g, "norm", "RMSNorm", {x, gamma}, "{\"eps\": 1e-5}");
            auto sg = gen(*g, "sig", "Sigmoid", {n});
            auto ad = gen(*g, "add", "Add", {row, sg});
            g->add_node_and_edge(std::make_shared<op::Result>(), {ad});
            pass::graph::DefaultKernelSelector sel;
            CONTAINS(sel.pick_first(n, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                     "nnf_rms_norm_f16(stream, input0, input1, output0, 8, 256, 1.000000000e-05f)");
            CONTAINS(sel.pick_first(sg, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(), "NNF_EW_SIGMOID, input0, nullptr");
            CONTAINS(sel.pick_first(ad, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                     "NNF_EW_ADD, input1, input0, output0, 8, 256, 1)");
        }
        {
            // Dot{transpose_B}(x, Dequantize(Wq, S, Z)) folds into one QuantDot that carries the block parameters; a
            // Dequantize with another consumer stays and has an emitter
            auto g = std::make_shared<graph::Graph>();
            auto x = param(*g, element::f16, Shape{M, H});
            auto w = cst(*g, element::u8, Shape{I, H / 2}, 0x31), sc = cst(*g, element::f16, Shape{I, H / 32}, 0x21);
            auto z = cst(*g, element::u8, Shape{I, H / 32 / 2}, 0x77);
            auto dq = gen(*g, "dq", "Dequantize", {w, sc, z}, "{\"bits\": 4, \"group_size\": 32, \"zero_point\": 0, \"has_zero_points\": true}");
            EXPECT(dq->get_output_shape(0) == (Shape{I, H}) && dq->get_output_element_type(0) == element::f16);
            auto d = gen(*g, "dot", "Dot", {x, dq}, "{\"transpose_B\": true}");
            EXPECT(d->get_output_shape(0) == (Shape{M, I}));
            g->add_node_and_edge(std::make_shared<op::Result>(), {d});
            g->add_node_and_edge(std::make_shared<op::Result>(), {dq});
            pass::graph::QuantEpilogueFusionPass fusion;
            EXPECT(fusion.run_on_graph(g) && fusion.fused == 1);
            EXPECT(count(g, "Dot") == 0 && count(g, "QuantDot") == 1 && count(g, "Dequantize") == 1);
            auto q = find(g, "QuantDot");
            auto& cfg = std::dynamic_pointer_cast<op::GenericOp>(q->get_op_ptr())->localOpConfig.getRoot();
            EXPECT(cfg["bits"].get<int>() == 4 && cfg["group_size"].get<int>() == 32 && cfg["has_zero_points"].get<bool>() &&
                   q->get_input_size() == 4 && q->get_input_shape(3) == (Shape{I, H / 32 / 2}));
            pass::graph::DefaultKernelSelector sel;
            CONTAINS(sel.pick_first(q, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                     "nnf_wna16_gemm(stream, input0, input1, input2, output0, 8, 384, 256, &quant, ");
            auto fu = sel.pick_first(find(g, "Dequantize"), ROCM_GPU).second->get_or_emit_source();
            CONTAINS(fu->body_unit->get_code(), "const nnf_quant quant = {4, 32, 0, input2};");
            CONTAINS(fu->body_unit->get_code(), "nnf_dequantize_f16(stream, input0, input1, output0, 384, 256, &quant)");
            // Dot validates like the reference's: operands of one element type
            bool threw = false;
            try
            {
                gen(*g, "bad", "Dot", {x, w}, "{\"transpose_B\": true}");
            }
            catch (const std::exception&)
            {
                threw = true;
            }
            EXPECT(threw);
        }
        {
            // the MLP block with blocks of 32 and a zero point per block: one FusedQuantMLP with the two zero-point tensors
            // behind its six inputs, emitted as one call that runs the nodes one after the other
            auto g = std::make_shared<graph::Graph>();
            auto x = param(*g, element::f16, Shape{M, H});
            auto gamma = cst(*g, element::f16, Shape{H}, 0x3c);
            const std::string qc = "{\"bits\": 4, \"group_size\": 32, \"zero_point\": 0, \"has_zero_points\": true}";
            auto wg = cst(*g, element::u8, Shape{I, H / 2}, 0x11), sg = cst(*g, element::f16, Shape{I, H / 32}, 0x21);
            auto zg = cst(*g, element::u8, Shape{I, H / 64}, 0x51);
            auto wu = cst(*g, element::u8, Shape{I, H / 2}, 0x12), su = cst(*g, element::f16, Shape{I, H / 32}, 0x22);
            auto zu = cst(*g, element::u8, Shape{I, H / 64}, 0x52);
            auto wd = cst(*g, element::u8, Shape{H, I / 2}, 0x13), sd = cst(*g, element::f16, Shape{H, I / 32}, 0x23);
            auto zd = cst(*g, element::u8, Shape{H, I / 64}, 0x53);
            auto n = gen(*g, "norm", "RMSNorm", {x, gamma});
            auto gate = gen(*g, "gate", "QuantDot", {n, wg, sg, zg}, qc);
            auto up = gen(*g, "up", "QuantDot", {n, wu, su, zu}, qc);
            auto h = gen(*g, "h", "Multiply", {up, gen(*g, "act", "Swish", {gate})});
            auto down = gen(*g, "down", "QuantDot", {h, wd, sd, zd}, qc);
            g->add_node_and_edge(std::make_shared<op::Result>(), {gen(*g, "out", "Add", {down, x})});
            pass::graph::QuantEpilogueFusionPass fusion;
            EXPECT(fusion.run_on_graph(g));
            EXPECT(count(g, "FusedQuantMLP") == 1 && count(g, "QuantDot") == 0 && count(g, "RMSNorm") == 0 && count(g, "Multiply") == 0);
            auto mlp = find(g, "FusedQuantMLP");
            EXPECT(mlp && mlp->get_input_size() == 8 && mlp->get_input_shape(6) == (Shape{2 * I, H / 64}) &&
                   mlp->get_input_shape(7) == (Shape{H, I / 64}));
            auto zc = std::dynamic_pointer_cast<op::Constant>(mlp->get_in_edge(6).src->get_op_ptr());
            EXPECT(zc && zc->get_data().front() == 0x51 && zc->get_data().back() == 0x52);
            pass::graph::DefaultKernelSelector sel;
            auto body = sel.pick_first(mlp, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code();
            CONTAINS(body, "const nnf_quant quant_gate_up = {4, 32, 0, input6};");
            CONTAINS(body, "const nnf_quant quant_down = {4, 32, 0, input7};");
            CONTAINS(body, "nnf_fused_mlp_wna16(stream, input0, input1, 1.000000000e-06f, input2, input3, input4, input5, output0, 8, 256, 384, &quant_gate_up, &quant_down, ");
        }
        {
            // bias (constant row) then residual (same shape) fold in that order; a second Add of a constant does not
            auto g = std::make_shared<graph::Graph>();
            auto x = param(*g, element::f16, Shape{M, H});
            auto r = param(*g, element::f16, Shape{M, I});
            auto w = cst(*g, element::u8, Shape{I, H / 2}, 1), s = cst(*g, element::f16, Shape{I, H / 128}, 2);
            auto b = cst(*g, element::f16, Shape{I}, 3), b2 = cst(*g, element::f16, Shape{I}, 4);
            auto d = gen(*g, "d", "QuantDot", {x, w, s});
            auto y = gen(*g, "y", "Add", {gen(*g, "yb", "Add", {d, b}), r});
            auto z = gen(*g, "z", "Add", {y, b2});
            g->add_node_and_edge(std::make_shared<op::Result>(), {z});
            pass::graph::QuantEpilogueFusionPass fusion;
            EXPECT(fusion.run_on_graph(g) && fusion.fused == 2);
            EXPECT(count(g, "QuantDot") == 1 && count(g, "Add") == 1);
            auto q = find(g, "QuantDot");
            auto& cfg = std::dynamic_pointer_cast<op::GenericOp>(q->get_op_ptr())->localOpConfig.getRoot();
            EXPECT(cfg["has_bias"].get<bool>() && cfg["has_residual"].get<bool>() && q->get_input_size() == 5);
            EXPECT(q->get_input_shape(3) == (Shape{I}) && q->get_input_shape(4) == (Shape{M, I}));
            // and the fused node still finds its emitter
            pass::graph::DefaultKernelSelector sel;
            auto fu = sel.pick_first(q, ROCM_GPU).second->get_or_emit_source();
            CONTAINS(fu->body_unit->get_code(), "nullptr, 1.000000000e-06f, input3, input4, NNF_ACT_NONE");
        }
        {
            // q / k / v read the same normalised activations: one 3N-row QuantDot and three Slices
            auto g = std::make_shared<graph::Graph>();
            auto x = param(*g, element::f16, Shape{M, H});
            auto gamma = cst(*g, element::f16, Shape{H}, 0x3c);
            auto n = gen(*g, "norm", "RMSNorm", {x, gamma});
            auto other = param(*g, element::f16, Shape{M, H});
            const size_t rows[3] = {128, 64, 64};
            for (int i = 0; i < 3; ++i)
            {
                auto w = cst(*g, element::u8, Shape{rows[i], H / 2}, (uint8_t)(0x40 + i));
                auto s = cst(*g, element::f16, Shape{rows[i], H / 128}, (uint8_t)(0x50 + i));
                g->add_node_and_edge(std::make_shared<op::Result>(), {gen(*g, "p" + std::to_string(i), "QuantDot", {n, w, s})});
            }
            // a QuantDot on other activations is left alone
            auto w = cst(*g, element::u8, Shape{32, H / 2}, 9), s = cst(*g, element::f16, Shape{32, H / 128}, 9);
            g->add_node_and_edge(std::make_shared<op::Result>(), {gen(*g, "lone", "QuantDot", {other, w, s})});
            pass::graph::QuantEpilogueFusionPass fusion;
            pass::graph::QuantGemmFusionPass merge;
            EXPECT(fusion.run_on_graph(g) && merge.run_on_graph(g) && merge.merged_groups == 1);
            EXPECT(count(g, "QuantDot") == 2 && count(g, "Slice") == 3 && count(g, "RMSNorm") == 0 && count(g, "Result") == 4);
            std::shared_ptr<graph::GNode> wide;
            std::vector<std::pair<int, int>> ranges;
            for (auto& node : g->get_ordered_ops())
            {
                if (node->get_op_type() == "QuantDot" && node->get_output_shape(0).back() == 256)
                    wide = node;
                if (node->get_op_type() == "Slice")
                {
                    auto& cfg = std::dynamic_pointer_cast<op::GenericOp>(node->get_op_ptr())->localOpConfig.getRoot();
                    ranges.push_back({cfg["begin"].get<int>(), cfg["end"].get<int>()});
                }
            }
            EXPECT(wide && wide->get_input_size() == 4 && wide->get_input_shape(1) == (Shape{256, H / 2}));
            EXPECT(ranges.size() == 3 && ranges[0] == std::make_pair(0, 128) && ranges[1] == std::make_pair(128, 192) &&
                   ranges[2] == std::make_pair(192, 256));
            auto wc = std::dynamic_pointer_cast<op::Constant>(wide->get_in_edge(1).src->get_op_ptr());
            EXPECT(wc && wc->get_data()[0] == 0x40 && wc->get_data()[128 * H / 2] == 0x41 && wc->get_data().back() == 0x42);
            // the Slice has an emitter: a strided device-to-device copy
            pass::graph::DefaultKernelSelector sel;
            auto sl = find(g, "Slice");
            CONTAINS(sel.pick_first(sl, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                     "hipMemcpy2DAsync(output0, 256, (const char*)input0 + 0, 512, 256, 8, hipMemcpyDeviceToDevice, stream)");
        }
    });

    // QuantDot with other block parameters than the specialised kernels': shapes, emitter, and that the fusion passes
    // leave such a node alone (only the 4-bit / 128 / scalar-zero-point product has fused forms)
    run_case("quant_dot_block_parameters", [] {
        auto cst = [](graph::Graph& g, const element::Type& t, const Shape& s) {
            std::vector<uint8_t> d(shape_size(s) * t.size(), 1);
            return g.add_node_and_edge(std::make_shared<op::Constant>(t, s, d.data()), graph::GNodeVector{});
        };
        auto quant_dot = [](graph::Graph& g, const graph::GNodeVector& in, const std::string& cfg) {
            return g.add_node_and_edge(std::make_shared<op::GenericOp>("qd", "QuantDot", op::OpConfig::any::parse(cfg)), in);
        };
        const size_t M = 4, N = 48, K = 320;
        pass::graph::DefaultKernelSelector sel;
        {
            // 8 bits, groups of 64, a zero point per (row, group): five groups of a row in five bytes
            auto g = std::make_shared<graph::Graph>();
            auto x = param(*g, element::f16, Shape{M, K});
            auto q = quant_dot(*g, {x, cst(*g, element::u8, Shape{N, K}), cst(*g, element::f16, Shape{N, K / 64}),
                                    cst(*g, element::u8, Shape{N, K / 64})},
                               "{\"bits\": 8, \"group_size\": 64, \"zero_point\": 0, \"has_zero_points\": true}");
            EXPECT(q->get_output_shape(0) == (Shape{M, N}) && q->get_output_element_type(0) == element::f16);
            const std::string body = sel.pick_first(q, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code();
            CONTAINS(body, "const nnf_quant quant = {8, 64, 0, input3};");
            CONTAINS(body, "nnf_wna16_gemm(stream, input0, input1, input2, output0, 4, 48, 320, &quant, nullptr, 0)");
        }
        {
            // 4 bits, groups of 32, scalar zero point; ten groups, and with a tensor five bytes of two zero points each
            auto g = std::make_shared<graph::Graph>();
            auto x = param(*g, element::f16, Shape{M, K});
            auto q = quant_dot(*g, {x, cst(*g, element::u8, Shape{N, K / 2}), cst(*g, element::f16, Shape{N, K / 32})},
                               "{\"group_size\": 32, \"zero_point\": 3}");
            CONTAINS(sel.pick_first(q, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code(),
                     "const nnf_quant quant = {4, 32, 3, nullptr};");
            bool threw = false;
            try
            {
                quant_dot(*g, {x, cst(*g, element::u8, Shape{N, K / 2}), cst(*g, element::f16, Shape{N, K / 32}),
                               cst(*g, element::u8, Shape{N, K / 32})},
                          "{\"group_size\": 32, \"has_zero_points\": true}");
            }
            catch (const CheckError&)
            {
                threw = true; // zero points of 4 bits come two to a byte: [N, 5]
            }
            EXPECT(threw);
            threw = false;
            try
            {
                quant_dot(*g, {x, cst(*g, element::u8, Shape{N, K / 2}), cst(*g, element::f16, Shape{N, K / 32})},
                          "{\"bits\": 8, \"group_size\": 32}"); // 8-bit weights are [N, K]
            }
            catch (const CheckError&)
            {
                threw = true;
            }
            EXPECT(threw);
        }
        {
            // 4-bit weights above 16 rows with K a multiple of 256: the tile GEMM's scratch memory comes with the call
            auto g = std::make_shared<graph::Graph>();
            auto x = param(*g, element::f16, Shape{128, 4096});
            auto q = quant_dot(*g, {x, cst(*g, element::u8, Shape{4096, 2048}), cst(*g, element::f16, Shape{4096, 64}),
                                    cst(*g, element::u8, Shape{4096, 32})},
                               "{\"group_size\": 64, \"has_zero_points\": true}");
            auto k = sel.pick_first(q, ROCM_GPU).second;
            const std::string body = k->get_or_emit_source()->body_unit->get_code();
            const size_t ws = nnf::workspace::wna16_gemm(128, 4096, 4096, 4, 64);
            EXPECT(ws > 0 && ws == nnf::workspace::plan_w4a16_sk(128, 4096, 4096, false, nnf::workspace::PLAN_CUS).bytes());
            CONTAINS(body, "const nnf_quant quant = {4, 64, 8, input3};");
            // ... through the entry point that takes the synchronisation words of the one-launch form (two per tile, 32 tiles
            // of 128 x 128, and two more: a second, persistent and zero-initialised tensor)
            EXPECT(k->m_context->tensors.size() == 2 && k->m_context->tensors[1]->size() == 320 &&
                   k->m_context->tensors[1]->is_persistent() && k->m_context->tensors[1]->is_memset());
            CONTAINS(body, "const nnf_plan plan = {0, 0, 0, " + k->m_context->tensors[1]->get_name() + ", 320, 0};");
            CONTAINS(body, "nnf_wna16_gemm_planned(stream, input0, input1, input2, output0, 128, 4096, 4096, &quant, &plan, ");
            CONTAINS(body, ", " + std::to_string(ws) + "));");
            EXPECT(body.find("&quant, nullptr") == std::string::npos);
            // 8-bit weights, K not a multiple of 256, 16 rows: the kernels that need none
            EXPECT(nnf::workspace::wna16_gemm(128, 4096, 4096, 8, 64) == 0 && nnf::workspace::wna16_gemm(128, 4096, 4096 + 128, 4, 64) == 0 &&
                   nnf::workspace::wna16_gemm(16, 4096, 4096, 4, 64) == 0 && nnf::workspace::wna16_gemm(128, 4096, 4096, 4, 16) == 0);
        }
        {
            // RMSNorm -> QuantDot(groups of 64) -> Add: both fold into the product (nnf_wna16_gemm_fused runs the nodes one
            // after the other inside one call), which keeps its block parameters
            auto g = std::make_shared<graph::Graph>();
            auto x = param(*g, element::f16, Shape{M, K});
            auto r = param(*g, element::f16, Shape{M, N});
            auto n = g->add_node_and_edge(std::make_shared<op::GenericOp>("norm", "RMSNorm", op::OpConfig::any()),
                                          {x, cst(*g, element::f16, Shape{K})});
            auto q = quant_dot(*g, {n, cst(*g, element::u8, Shape{N, K / 2}), cst(*g, element::f16, Shape{N, K / 64})},
                               "{\"group_size\": 64}");
            auto y = g->add_node_and_edge(std::make_shared<op::GenericOp>("y", "Add", op::OpConfig::any()), {q, r});
            g->add_node_and_edge(std::make_shared<op::Result>(), {y});
            pass::graph::QuantEpilogueFusionPass fusion;
            pass::graph::QuantGemmFusionPass merge;
            EXPECT(fusion.run_on_graph(g));
            EXPECT(fusion.fused >= 2); // (a rewrite that a later one of the same sweep supersedes counts as well)
            EXPECT(merge.run_on_graph(g) && merge.merged_groups == 0);
            size_t norms = 0, adds = 0;
            std::shared_ptr<graph::GNode> fusedq;
            for (auto& node : g->get_ordered_ops())
            {
                norms += node->get_op_type() == "RMSNorm";
                adds += node->get_op_type() == "Add";
                if (node->get_op_type() == "QuantDot")
                    fusedq = node;
            }
            EXPECT(norms == 0 && adds == 0 && fusedq != nullptr);
            const std::string body = sel.pick_first(fusedq, ROCM_GPU).second->get_or_emit_source()->body_unit->get_code();
            CONTAINS(body, "const nnf_quant quant = {4, 64, 8, nullptr};");
            CONTAINS(body, "nnf_wna16_gemm_fused(stream, input0, input1, input2, output0, " + std::to_string(M) + ", " + std::to_string(N) +
                               ", " + std::to_string(K) + ", &quant, input3, 1.000000000e-06f, nullptr, input4, NNF_ACT_NONE, ");
        }
    });

    // the host arithmetic that picks a kernel variant for a shape and sizes its LDS / workspace
    run_case("kernel_plans", [] {
        namespace ws = nnf::workspace;
        // one activation row: the row-streaming kernel
        {
            auto p = ws::plan_w4a16_rows(1, 4096, 4096, 256);
            EXPECT(p.seg == 2 && p.kshift == 0 && p.depth == 2);
            p = ws::plan_w4a16_rows(1, 22016, 4096, 256);
            EXPECT(p.seg == 2 && p.kshift == 0 && p.depth == 2);
            p = ws::plan_w4a16_rows(1, 4096, 11008, 256);
            EXPECT(p.seg == 3 && p.kshift == 1 && p.depth == 2);
            p = ws::plan_w4a16_rows(1, 8192, 8192, 256);
            EXPECT(p.seg == 2 && p.kshift == 1);
            p = ws::plan_w4a16_rows(1, 152064, 2048, 256);
            EXPECT(p.seg == 1 && p.kshift == 0 && p.depth == 4);
            // fewer rows than wavefronts: no prefetch beyond the first row
            EXPECT(ws::plan_w4a16_rows(1, 300, 1024, 256).depth == 1);
            EXPECT(ws::rows_grid(40, 256) == 40 && ws::rows_grid(4096, 256) == 256);
            // not this kernel's shapes
            EXPECT(ws::plan_w4a16_rows(2, 4096, 4096, 256).seg == 0);
            EXPECT(ws::plan_w4a16_rows(1, 4096, 128, 256).seg == 0);
            EXPECT(ws::plan_w4a16_rows(1, 4096, 4096 + 128, 256).seg == 0);
            EXPECT(ws::plan_w4a16_rows(1, 4096, 32768, 256).seg == 0);
            EXPECT(ws::plan_w4a16_rows(1, 0, 4096, 256).seg == 0);
            const int ns[] = {1, 7, 40, 256, 300, 513, 4096, 5000, 12288, 22016, 32000, 80000, 152064, 1000000};
            for (int n : ns)
                for (int k = 1024; k <= 16384; k += 256)
                {
                    p = ws::plan_w4a16_rows(1, n, k, 256);
                    if (p.seg == 0)
                        continue; // (a very tall matrix with long rows: the workgroup's scales do not fit)
                    const int grid = ws::rows_grid(n, 256);
                    EXPECT(p.seg >= 1 && p.seg <= 3 && p.kshift >= 0 && p.kshift <= 3 && p.depth >= 1 && p.depth <= 4);
                    EXPECT(((size_t)p.seg << p.kshift) * 1024 >= (size_t)k / 2);        // the segments cover a row
                    EXPECT(((size_t)p.seg << p.kshift) * 1024 < (size_t)k / 2 + 1024 * (size_t)(1 << p.kshift)); // tightly
                    EXPECT(p.lds_bytes(n, k, grid) <= ws::LDS_BYTES_PER_CU);
                    // the first `depth` rows of every wavefront are fixed: they must exist
                    EXPECT(p.depth == 1 || p.depth * (ws::ROWS_WAVES >> p.kshift) <= n / grid);
                }
            EXPECT(ws::plan_w4a16_rows(1, 1000000, 16384, 256).seg == 0);
            // other block parameters: groups of 32 / 64 (more scales per row) and zero-point tensors (256 bytes more per
            // ring slot and 64 groups, a second constant per unit of activations); not with the SiLU-gate
            p = ws::plan_w4a16_rows(1, 4096, 4096, 256, 0, false, 5, true);
            EXPECT(p.seg == 2 && p.kshift == 0 && p.depth == 2);
            EXPECT(p.lds_bytes(4096, 4096, 256, false, 5, true) ==
                   (size_t)8 * 2 * (2 * 1024 + 256) + 516 * 16 + 2 * 516 * 4 + 5120 + 17 * 4 + 64);
            EXPECT(ws::plan_w4a16_rows(1, 4096, 11008, 256, 0, false, 5, true).seg == 3);
            EXPECT(ws::plan_w4a16_rows(1, 4096, 4096, 256, 0, false, 4, false).seg == 0);
            EXPECT(ws::plan_w4a16_rows(1, 4096, 4096, 256, 0, false, 8, false).seg == 0);
            EXPECT(ws::plan_w4a16_rows(1, 4096, 4096, 256, 0, true, 6, false).seg == 0);
            EXPECT(ws::plan_w4a16_rows(1, 4096, 4096, 256, 0, true, 7, true).seg == 0);
            for (int n : ns)
                for (int k = 1024; k <= 16384; k += 1280)
                    for (int gs = 5; gs <= 7; ++gs)
                    {
                        p = ws::plan_w4a16_rows(1, n, k, 256, 0, false, gs, true);
                        if (p.seg == 0)
                            continue;
                        const int grid = ws::rows_grid(n, 256);
                        EXPECT(p.lds_bytes(n, k, grid, false, gs, true) <= ws::LDS_BYTES_PER_CU);
                        EXPECT(p.lds_bytes(n, k, grid, false, gs, true) > p.lds_bytes(n, k, grid, false, gs, false));
                        EXPECT(p.depth == 1 || p.depth * (ws::ROWS_WAVES >> p.kshift) <= n / grid);
                    }
        }
        // a few rows with other block parameters: K = 2048 / 4096 / 8192, whole words of scales per step and wavefront
        {
            EXPECT(ws::w4a16_mrows_q_fits(16, 8192, 8192, 6, true, 256));
            EXPECT(ws::w4a16_mrows_q_fits(2, 4096, 4096, 5, false, 256));
            EXPECT(ws::w4a16_mrows_q_fits(8, 300, 2048, 6, true, 256));
            EXPECT(!ws::w4a16_mrows_q_fits(8, 300, 2048, 7, true, 256)); // half a word of scales
            EXPECT(!ws::w4a16_mrows_q_fits(1, 4096, 4096, 5, false, 256) && !ws::w4a16_mrows_q_fits(33, 4096, 4096, 5, false, 256));
            // 17 .. 32 rows: two blocks of rows in registers, up to K = 4096 (no workspace: not the tile GEMM)
            EXPECT(ws::w4a16_mrows_q_fits(17, 4096, 4096, 5, false, 256) && ws::w4a16_mrows_q_fits(32, 12288, 2048, 6, true, 256));
            EXPECT(!ws::w4a16_mrows_q_fits(17, 8192, 8192, 5, false, 256));
            EXPECT(ws::w4a16_mrows_q_lds_bytes(4096, 32, 1, 6, false) == 32768 + 4096 + 65536);
            EXPECT(ws::wna16_gemm(32, 4096, 4096, 4, 64) == 0 && ws::wna16_gemm(32, 8192, 8192, 4, 64) > 0 &&
                   ws::wna16_gemm(33, 4096, 4096, 4, 64) > 0);
            EXPECT(!ws::w4a16_mrows_q_fits(8, 4096, 6144, 5, false, 256) && !ws::w4a16_mrows_q_fits(8, 4096, 11008, 5, false, 256));
            EXPECT(!ws::w4a16_mrows_q_fits(8, 4096, 4096, 4, false, 256) && !ws::w4a16_mrows_q_fits(8, 8, 4096, 5, false, 256));
            // ring 8 x 2 x 4 KiB, scales and zero points 8 x 2 x (2 + 2) x 256, then the larger of partial tiles 16 KiB + parked tiles
            // and the 64 KiB through which the activations arrive
            EXPECT(ws::w4a16_mrows_q_lds_bytes(8192, 16, 2, 5, true) == 65536 + 16384 + 65536);
            EXPECT(ws::w4a16_mrows_q_lds_bytes(4096, 16, 1, 6, false) == 32768 + 4096 + 65536);
            EXPECT(!ws::w4a16_mrows_q_fits(16, 1000000, 8192, 5, true, 256)); // the parked sums do not fit
        }
        // ... with a run-time K: one piece up to 8192 where most of what is fetched counts, ranges of at most 32 blocks above
        {
            auto p = ws::w4a16_mrows_q_any_plan(16, 4096, 11008, 7, true, 256);
            EXPECT(p.ranges == 3 && p.range_blocks == 30 && p.gw == 2);
            EXPECT(ws::wna16_gemm(16, 4096, 11008, 4, 128) == (size_t)3 * 16 * 4096 * 4);
            p = ws::w4a16_mrows_q_any_plan(8, 4096, 5120, 5, false, 256);
            EXPECT(p.ranges == 1 && p.gw == 3 && p.range_blocks == 40);
            EXPECT(ws::wna16_gemm(8, 4096, 5120, 4, 32) == 0);
            EXPECT(ws::w4a16_mrows_q_any_plan(8, 4096, 7168, 6, true, 256).gw == 4);
            EXPECT(ws::w4a16_mrows_q_any_plan(8, 4096, 2304, 6, true, 256).ranges == 0); // 18 of 32 fetched blocks count
            EXPECT(ws::w4a16_mrows_q_any_plan(17, 4096, 11008, 6, true, 256).ranges == 0);
            EXPECT(ws::w4a16_mrows_q_any_plan(8, 4096, 11008 + 128, 6, true, 256).ranges == 0);
            p = ws::w4a16_mrows_q_any_plan(4, 8192, 28672, 7, true, 256);
            EXPECT(p.ranges == 7 && p.range_blocks == 32 && p.gw == 2);
            // scales of a step: groups of 128: gw / 2 + 1 words a row; 32: gw * 2 words (two loads from gw = 3 on)
            EXPECT(ws::w4a16_mrows_q_any_lds_bytes(2, 16, 1, 7, true) == 32768 + 8 * 2 * 512 + 65536);
            EXPECT(ws::w4a16_mrows_q_any_lds_bytes(4, 16, 1, 5, false) == 65536 + 8 * 2 * 512 + 65536);
        }
        // M <= 16: one workgroup holds the activations, or K is cut into ranges
        {
            for (int m = 1; m <= 16; ++m)
                EXPECT(ws::w4a16_skinny_fits(m, 22016, 4096));
            EXPECT(ws::w4a16_skinny_fits(7, 8192, 8192) && !ws::w4a16_skinny_fits(8, 8192, 8192));
            EXPECT(ws::w4a16_skinny_ksplits(16, 8192, 8192) == 2 && ws::w4a16_skinny_ksplits(7, 8192, 8192) == 0);
            // K that does not divide into equal ranges of a multiple of 1024: a shorter last range
            EXPECT(ws::w4a16_skinny_split_range(16, 8192, 8192 + 128) == 3072 && ws::w4a16_skinny_ksplits(16, 8192, 8192 + 128) == 3);
            EXPECT(ws::w4a16_skinny_split_range(8, 4096, 11008) == 4096 && ws::w4a16_skinny_ksplits(8, 4096, 11008) == 3);
            EXPECT(ws::w4a16_skinny_ksplits(16, 4096, 13824) == 4 && ws::w4a16_skinny_ksplits(4, 4096, 11008) == 0);
            EXPECT(ws::skinny_split_bytes(8, 4096, 11008) == (size_t)3 * 8 * 4096 * 4);
            EXPECT(!ws::w4a16_skinny_fits(17, 4096, 4096) && !ws::w4a16_skinny_fits(4, 4096, 4096 + 64) &&
                   !ws::w4a16_skinny_fits(4, 8, 4096));
            // weights addressed with 32-bit offsets
            EXPECT(!ws::w4a16_skinny_fits(1, 1 << 20, 8192) && ws::w4a16_skinny_fits(1, 1 << 19, 8192));
            // one launch, no scratch memory, where a row-streaming kernel serves the shape; ranges of K and shared tiles park sums
            EXPECT(ws::w4a16_gemm(1, 4096, 4096, 128) == 0 && ws::w4a16_gemm(16, 12288, 4096, 128) == 0 &&
                   ws::w4a16_gemm(7, 8192, 8192, 128) == 0);
            // 8 .. 16 rows at K = 8192 (up to 8192 weight rows): two ranges of K (half the activations per workgroup)
            EXPECT(ws::w4a16_gemm(16, 8192, 8192, 128) == (size_t)2 * 16 * 8192 * 4 && ws::w4a16_gemm(8, 4096, 8192, 128) == (size_t)2 * 8 * 4096 * 4 &&
                   ws::w4a16_gemm(16, 16384, 8192, 128) == 0 && ws::w4a16_gemm(16, 28672, 8192, 128) == 0);
            EXPECT(ws::route_w4a16(16, 8192, 8192, false, true, false, 256).kind == ws::W4A16Route::MROWS &&
                   ws::route_w4a16(16, 4096, 8192, true, false, false, 256).kind == ws::W4A16Route::MROWS);
            EXPECT(ws::mrows_split_adds_in_launch(8192, 2, 256) && ws::mrows_split_adds_in_launch(4096, 3, 256) &&
                   !ws::mrows_split_adds_in_launch(28672, 2, 256));
            EXPECT(ws::w4a16_gemm(16, 4096, 11008, 128) == (size_t)3 * 16 * 4096 * 4 && ws::w4a16_gemm(128, 8192, 8192, 128) > 0);
            // the decode route of a fused MLP block: the row-streaming kernels take the RMSNorm weight, the gate product and
            // the residual themselves: rstd is the only scratch of the first product, the second needs none
            for (int m : {1, 16, 32})
            {
                const auto up = ws::route_w4a16(m, 11008, 4096, true, true, false, 256);
                EXPECT(up.kind == (m == 1 ? ws::W4A16Route::ROWS : ws::W4A16Route::MROWS) && up.partial_bytes == 0 &&
                       up.rms_bytes == 256);
                const auto down = ws::route_w4a16(m, 4096, 11008, false, false, true, 256);
                EXPECT(down.kind == (m == 1 ? ws::W4A16Route::ROWS : ws::W4A16Route::MROWS_SPLIT));
                EXPECT(down.partial_bytes == (m == 1 ? 0 : (size_t)3 * m * 4096 * 4) && down.rms_bytes == 0);
                EXPECT(ws::fused_mlp_w4a16(m, 4096, 11008, 128) == 256 + ws::align256((size_t)m * 11008 * 2) + down.partial_bytes);
            }
            // (four rows of K = 11008 still fit one workgroup's LDS: the MFMA GEMV kernel in one launch, its products in
            // scratch when the residual is the output buffer)
            EXPECT(ws::route_w4a16(4, 4096, 11008, false, false, true, 256).kind == ws::W4A16Route::SKINNY &&
                   ws::route_w4a16(4, 4096, 11008, false, false, true, 256).partial_bytes == (size_t)4 * 4096 * 2 &&
                   ws::route_w4a16(4, 4096, 11008, false, false, false, 256).partial_bytes == 0);
            // one family of kernels only: the MFMA GEMV kernel reads normalised activations and leaves gate | up in scratch
            {
                const auto r = ws::route_w4a16(8, 11008, 4096, true, true, false, 256, 2);
                EXPECT(r.kind == ws::W4A16Route::SKINNY && r.via_scratch && r.partial_bytes == (size_t)8 * 22016 * 2 &&
                       r.rms_bytes == (size_t)8 * 4096 * 2);
                EXPECT(ws::route_w4a16(64, 4096, 4096, false, false, false, 256, 2).kind == ws::W4A16Route::NONE);
                EXPECT(ws::route_w4a16(64, 4096, 4096, false, false, false, 256, 4).kind == ws::W4A16Route::NONE);
                EXPECT(ws::route_w4a16(64, 4096, 4096, false, false, false, 256, 0).kind == ws::W4A16Route::TILE);
            }
            for (int k = 128; k <= 16384; k += 128)
            {
                const auto p = ws::plan_w4a16_skinny(4, k);
                EXPECT(p.cps >= 1 && p.ks >= 1 && p.ks <= 16 && p.cps * p.h * p.ks >= k / 128);
            }
        }
        // W8A8, M <= 16
        for (int k = 128; k <= 16384; k += 128)
        {
            const auto p = ws::plan_w8a8_skinny(1, k);
            EXPECT(p.cps >= 1 && p.ks >= 1 && p.ks <= 16 && (p.kh == 1 || p.kh == 2 || p.kh == 4 || p.kh == 8));
            EXPECT(p.cps * p.kh * p.ks >= k / 64 && p.cps * p.kh * (p.ks - 1) < k / 64);
            EXPECT(ws::w8a8_skinny_fits(1, k) && ws::w8a8_gemm(1, 4096, k) == 0);
        }
        EXPECT(!ws::w8a8_skinny_fits(16, 8192) && ws::w8a8_gemm(16, 8192, 8192) > 0);
        // the row-streaming kernel over two ranges of K: 8 .. 32 rows, K from 8192 in multiples of 512, at most four tiles
        // per workgroup of a range; the workspace query covers the ranges' int32 sums
        EXPECT(ws::w8a8_mrows_ranges(8, 4096, 8192, 256) == 2 && ws::w8a8_mrows_ranges(32, 8192, 8192, 256) == 2 &&
               ws::w8a8_mrows_ranges(16, 4096, 14336, 256) == 2);
        EXPECT(ws::w8a8_mrows_ranges(7, 4096, 8192, 256) == 1 && ws::w8a8_mrows_ranges(32, 8192, 4096, 256) == 1 &&
               ws::w8a8_mrows_ranges(32, 8208, 8192, 256) == 1 && ws::w8a8_mrows_ranges(16, 4096, 11008, 256) == 1);
        EXPECT(ws::w8a8_mrows_ranges_bytes(8, 4096, 8192, 256) == (size_t)2 * 8 * 4096 * 4 && ws::w8a8_gemm(8, 4096, 8192) >= (size_t)2 * 8 * 4096 * 4);
        // fp16 x int4 tile GEMM: the (tile, superstep) units are split evenly over at most one workgroup per CU; a
        // workgroup parks at most two partial tiles; whole tiles need no workspace
        {
            const int ms[] = {17, 64, 128, 256, 1024, 4096};
            for (int m : ms)
                for (int gate = 0; gate < 2; ++gate)
                {
                    const auto p = ws::plan_w4a16_sk(m, 8192, 8192, gate != 0, 256);
                    EXPECT(p.supersteps == 32 && p.units == (long long)p.tiles_m * p.tiles_n * 32);
                    EXPECT(p.grid >= 1 && p.grid <= 256 && p.units / p.grid >= 2);
                    EXPECT(p.tiles_m * p.tile_rows >= m && (p.tiles_m - 1) * p.tile_rows < m);
                    EXPECT(p.slots == 0 || p.slots == p.grid || p.slots == 2 * p.grid);
                    // tiles of 128 columns for the plain product up to 1536 rows (not for 32-row tiles), else 256 weight rows
                    EXPECT(p.tile_weight_rows == ((gate || m <= 32 || m > 1536) ? 256 : 128));
                    EXPECT(p.tiles_n == 8192 / ((gate || p.tile_weight_rows == 128) ? 128 : 256));
                    EXPECT(p.bytes() == (size_t)p.slots * p.tile_rows * p.tile_weight_rows * 4);
                    // every unit has exactly one owner, and owners follow each other
                    long long covered = 0;
                    for (int v = 0; v < p.grid; ++v)
                        covered += ((long long)(v + 1) * p.units) / p.grid - ((long long)v * p.units) / p.grid;
                    EXPECT(covered == p.units);
                }
            const auto big = ws::plan_w4a16_sk(4096, 8192, 8192, false, 256);
            EXPECT(big.tile_rows == 256 && big.grid == 256 && big.slots == 0 && big.bytes() == 0);
            EXPECT(ws::plan_w4a16_sk(128, 8192, 8192, false, 256).slots > 0);
            // 256 rows where M fills them to within an eighth, else 128; what a caller fixes is kept
            EXPECT(ws::plan_w4a16_sk(1024, 8192, 8192, false, 256).tile_rows == 256 && ws::plan_w4a16_sk(300, 8192, 8192, false, 256).tile_rows == 128);
            EXPECT(ws::plan_w4a16_sk(480, 8192, 8192, false, 256).tile_rows == 256 && ws::plan_w4a16_sk(100, 8192, 8192, false, 256).tile_rows == 128);
            const auto forced = ws::plan_w4a16_sk(1024, 8192, 8192, false, 256, 128, 0, 256);
            EXPECT(forced.tile_rows == 128 && forced.tile_weight_rows == 256 && forced.tiles_n == 32);
            EXPECT(ws::plan_w4a16_sk(1024, 8192, 8192, true, 256, 128, 0, 128).tile_weight_rows == 256); // SiLU-gate: full tiles
            EXPECT(ws::plan_w4a16_sk(4096, 8192, 8192, false, 256, 0, 0, 128).tile_weight_rows == 256);  // width alone: the plan's
            // K = 128 * odd: the last superstep of a tile holds one group
            EXPECT(ws::plan_w4a16_sk(64, 512, 384, false, 256).supersteps == 2);
        }
    });

    printf("%s (%d failure%s)\n", g_failures ? "FAILED" : "OK", g_failures, g_failures == 1 ? "" : "s");
    return g_failures ? 1 : 0;
}
