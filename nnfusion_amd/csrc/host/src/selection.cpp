// Device dispatch, kernel selection and the graph visitor.
#include "nnfusion/core/IR/instruction.hpp"
#include "nnfusion/core/operators/generic_op/generic_op.hpp"
#include "nnfusion/engine/pass/graph/kernel_selection.hpp"

#include <algorithm>

namespace nnfusion
{
    namespace pass
    {
        namespace graph
        {
            using namespace nnfusion::kernels;

            bool DefaultGNodeDeviceDispatcher::run_on_graph(std::shared_ptr<nnfusion::graph::Graph>& graph)
            {
                for (auto& node : graph->get_nodes())
                {
                    if (!(*node)["DeviceType"].is_valid())
                        (*node)["DeviceType"] = m_device;
                    if (!(*node)["DeviceID"].is_valid())
                        (*node)["DeviceID"] = 0;
                }
                return true;
            }

            namespace
            {
                // Emitter around an inline kernel string declared with OpConfig::cuda_kernel / cpu_kernel.
                class CustomInlineEmitter : public KernelEmitter
                {
                public:
                    CustomInlineEmitter(std::shared_ptr<KernelContext> ctx, const std::string& type)
                        : KernelEmitter(ctx, type)
                    {
                    }
                    LanguageUnit_p emit_function_body() override
                    {
                        auto gop = std::dynamic_pointer_cast<op::GenericOp>(m_context->op);
                        if (!gop)
                            return nullptr;
                        auto dev = get_device_str(get_device_type());
                        auto it = gop->localOpConfig.f_kernel_funcs.find(dev);
                        if (it == gop->localOpConfig.f_kernel_funcs.end())
                            return nullptr;
                        std::string code = it->second(m_context->gnode);
                        if (code.empty())
                            return nullptr;
                        LanguageUnit_p lu(new LanguageUnit(get_function_name()));
                        *lu << code;
                        return lu;
                    }
                    LanguageUnit_p emit_dependency() override
                    {
                        return LanguageUnit_p(new LanguageUnit(get_function_name() + "_dep"));
                    }
                };

                std::shared_ptr<KernelEmitter> make_custom_cuda(std::shared_ptr<KernelContext> ctx)
                {
                    return std::make_shared<CustomInlineEmitter>(ctx, "cuda");
                }
                std::shared_ptr<KernelEmitter> make_custom_cpu(std::shared_ptr<KernelContext> ctx)
                {
                    return std::make_shared<CustomInlineEmitter>(ctx, "cpu");
                }
            } // namespace

            bool DefaultKernelSelector::register_custom_kernel(const std::string& op_name, NNFusion_DeviceType devtype)
            {
                auto& configs = op::get_op_configs();
                auto it = configs.find(op_name);
                if (it == configs.end())
                    return false;
                // an inline CUDA string also serves ROCM_GPU nodes in the reference; this build emits HIP
                // only through registered emitters, so only exact device matches are registered
                NNFusion_DeviceType reg_dev = devtype;
                if (it->second.f_kernel_funcs.find(get_device_str(reg_dev)) == it->second.f_kernel_funcs.end())
                    return false;
                for (auto& r : KernelRegistry::Global()->FindKernelRegistrations(op_name, reg_dev, element::f32))
                    if (r->m_tag == "custom")
                        return true; // registered earlier
                KernelRegistrar registrar(op_name,
                                          Name(op_name)
                                              .Device(reg_dev)
                                              .TypeConstraint(element::f32)
                                              .Tag("custom")
                                              .Priority(10)
                                              .KernelFactory(reg_dev == GENERIC_CPU ? make_custom_cpu : make_custom_cuda)
                                              .Build());
                return true;
            }

            DefaultKernelSelector::Result DefaultKernelSelector::pick_first(std::shared_ptr<nnfusion::graph::GNode> gnode,
                                                                            NNFusion_DeviceType devtype)
            {
                std::shared_ptr<KernelContext> ctx(new KernelContext(gnode));
                register_custom_kernel(gnode->get_op_type(), devtype);
                auto regs = KernelRegistry::Global()->FindKernelRegistrations(gnode->get_op_type(), devtype, element::f32);
                if (devtype == ROCM_GPU)
                    for (auto& r : KernelRegistry::Global()->FindKernelRegistrations(gnode->get_op_type(), CUDA_GPU, element::f32))
                        regs.push_back(r);

                auto effective = [&](const std::shared_ptr<const KernelRegistration>& r) {
                    size_t prio = r->m_priority;
                    // an un-tuned "antares" registration ranks just above the reference kernels
                    if (r->m_tag == "antares")
                        prio = 1;
                    return prio + (r->m_device_type == devtype ? 1 : 0);
                };
                std::stable_sort(regs.begin(), regs.end(),
                                 [&](const std::shared_ptr<const KernelRegistration>& x,
                                     const std::shared_ptr<const KernelRegistration>& y) {
                                     size_t px = effective(x), py = effective(y);
                                     if (px != py)
                                         return px > py;
                                     return x->m_factory(ctx)->get_kernel_type() < y->m_factory(ctx)->get_kernel_type();
                                 });
                for (auto& r : regs)
                {
                    auto kernel = r->m_factory(ctx);
                    // constants are materialised by the code generator, not by an emitted function
                    if (gnode->is_constant() || kernel->get_or_emit_source())
                        return std::make_pair(devtype, kernel);
                }
                NNFUSION_LOG(ERROR) << "No valid kernel found:" << gnode->get_name() << "(op type: " << gnode->get_op_type()
                                    << ", dev type: " << get_device_str(devtype) << ")";
                return std::make_pair(devtype, KernelEmitter::Pointer());
            }

            bool DefaultKernelSelector::run_on_graph(std::shared_ptr<nnfusion::graph::Graph>& graph)
            {
                for (auto& node : graph->get_nodes())
                {
                    if ((*node)["Kernel_Selection_Result"].is_valid())
                        continue;
                    NNFUSION_CHECK((*node)["DeviceType"].is_valid())
                        << "GNode DeviceType should be assigned before this pass: " << node->get_name();
                    auto dev = (*node)["DeviceType"].as<NNFusion_DeviceType>();
                    NNFUSION_CHECK(dev != UNKNOWN);
                    if (node->is_parameter() || node->is_constant() || node->is_output())
                        continue; // tensor ops carry no kernel in this build
                    auto ans = pick_first(node, dev);
                    if (ans.second != nullptr)
                        (*node)["Kernel_Selection_Result"] = ans;
                }
                return true;
            }

            // ---- ProfilingBasedKernelSelector -----------------------------------------------------------------
            std::vector<KernelEmitter::Pointer>
                ProfilingBasedKernelSelector::candidates(std::shared_ptr<nnfusion::graph::GNode> gnode,
                                                         NNFusion_DeviceType devtype)
            {
                std::vector<KernelEmitter::Pointer> out;
                if (gnode->is_constant() || gnode->is_parameter() || gnode->is_output())
                    return out;
                auto regs = KernelRegistry::Global()->FindKernelRegistrations(gnode->get_op_type(), devtype, element::f32);
                if (devtype == ROCM_GPU)
                    for (auto& r : KernelRegistry::Global()->FindKernelRegistrations(gnode->get_op_type(), CUDA_GPU, element::f32))
                        regs.push_back(r);
                std::stable_sort(regs.begin(), regs.end(),
                                 [](const std::shared_ptr<const KernelRegistration>& x,
                                    const std::shared_ptr<const KernelRegistration>& y) { return x->m_priority > y->m_priority; });
                for (auto& r : regs)
                {
                    std::shared_ptr<KernelContext> ctx(new KernelContext(gnode)); // emitters may add scratch tensors
                    auto kernel = r->m_factory(ctx);
                    if (kernel->get_or_emit_source())
                        out.push_back(kernel);
                }
                return out;
            }

            std::vector<profiler::ProfilingContext::Pointer>
                ProfilingBasedKernelSelector::contexts(std::shared_ptr<nnfusion::graph::GNode> gnode,
                                                       NNFusion_DeviceType devtype, profiler::HipDefaultRuntime& runtime)
            {
                std::vector<profiler::ProfilingContext::Pointer> out;
                for (auto& k : candidates(gnode, devtype))
                {
                    auto pc = std::make_shared<profiler::ProfilingContext>(k);
                    pc->warmup_times = warmup_times;
                    pc->runtime_times = runtime_times;
                    pc->working_dir = working_dir;
                    if (runtime.codegen(pc))
                        out.push_back(pc);
                }
                return out;
            }

            namespace
            {
                // deterministic bytes; fp16 tensors get finite values of magnitude below two
                void fill_blob(std::vector<uint8_t>& blob, const element::Type& type, uint64_t seed)
                {
                    uint64_t x = seed * 0x9E3779B97F4A7C15ull + 0x2545F4914F6CDD1Dull;
                    for (size_t i = 0; i + 1 < blob.size() + 1; i += 2)
                    {
                        x ^= x << 13, x ^= x >> 7, x ^= x << 17;
                        uint16_t v = (uint16_t)(x >> 24);
                        if (type == element::f16)
                            v &= 0xBBFF;
                        else if (type == element::f32)
                            v = (i & 2) ? (uint16_t)(0x3A00 | (v & 0x80FF)) : v; // high half: sign, exponent ~2^-11
                        blob[i] = (uint8_t)v;
                        if (i + 1 < blob.size())
                            blob[i + 1] = (uint8_t)(v >> 8);
                    }
                }
            } // namespace

            ProfilingBasedKernelSelector::Result
                ProfilingBasedKernelSelector::profiling_best(std::shared_ptr<nnfusion::graph::GNode> gnode,
                                                             NNFusion_DeviceType devtype, profiler::HipDefaultRuntime& runtime,
                                                             std::vector<Timing>* timings,
                                                             std::vector<std::vector<uint8_t>>* outputs)
            {
                auto pcs = contexts(gnode, devtype, runtime);
                // nothing to choose between (the reference skips nodes with a single registration)
                if (pcs.size() < 2)
                    return std::make_pair(devtype, KernelEmitter::Pointer());
                if (prepare_only)
                {
                    for (auto& pc : pcs)
                        NNFUSION_CHECK(runtime.compile(pc)) << "kernel selection: cannot build the harness of "
                                                            << pc->kernel->get_function_name();
                    return std::make_pair(devtype, KernelEmitter::Pointer());
                }
                KernelEmitter::Pointer best;
                double best_ms = -1.0;
                for (auto& pc : pcs)
                {
                    auto& ctx = pc->kernel->m_context;
                    std::vector<std::vector<uint8_t>> in(ctx->inputs.size()), out(ctx->outputs.size());
                    std::vector<void*> in_p, out_p;
                    for (size_t i = 0; i < in.size(); ++i)
                    {
                        in[i].resize(std::max<size_t>(ctx->inputs[i]->size(), 2));
                        fill_blob(in[i], ctx->inputs[i]->get_element_type(), i + 1);
                        in_p.push_back(in[i].data());
                    }
                    for (size_t i = 0; i < out.size(); ++i)
                    {
                        out[i].assign(std::max<size_t>(ctx->outputs[i]->size(), 2), 0);
                        out_p.push_back(out[i].data());
                    }
                    const double ms = runtime.execute(pc, in_p.data(), out_p.data());
                    NNFUSION_LOG(INFO) << "Kernel Emitter " << pc->kernel->get_kernel_type() << " time cost(ms): " << ms;
                    if (timings)
                        timings->push_back(Timing{pc->kernel->get_kernel_type(), ms});
                    if (ms < 0)
                        continue;
                    if (outputs && !out.empty())
                        outputs->push_back(out[0]);
                    if (best_ms < 0 || ms < best_ms)
                    {
                        best_ms = ms;
                        best = pc->kernel;
                    }
                }
                return std::make_pair(devtype, best);
            }

            bool ProfilingBasedKernelSelector::run_on_graph(std::shared_ptr<nnfusion::graph::Graph>& graph,
                                                            profiler::HipDefaultRuntime& runtime)
            {
                if (!enable)
                    return true;
                static const std::vector<std::string> white_list{"QuantDot"};
                for (auto& node : graph->get_nodes())
                {
                    if (std::find(white_list.begin(), white_list.end(), node->get_op_type()) == white_list.end())
                        continue;
                    NNFUSION_CHECK((*node)["DeviceType"].is_valid())
                        << "GNode DeviceType should be assigned before this pass: " << node->get_name();
                    auto dev = (*node)["DeviceType"].as<NNFusion_DeviceType>();
                    if (dev != ROCM_GPU)
                        continue;
                    const std::string id = KernelContext(node).generate_identifier();
                    auto known = m_best_type.find(id);
                    if (known != m_best_type.end())
                    {
                        for (auto& k : candidates(node, dev))
                            if (k->get_kernel_type() == known->second)
                                (*node)["Kernel_Selection_Result"] = std::make_pair(dev, k);
                        continue;
                    }
                    auto ans = profiling_best(node, dev, runtime);
                    if (ans.second != nullptr)
                    {
                        m_best_type[id] = ans.second->get_kernel_type();
                        (*node)["Kernel_Selection_Result"] = ans;
                    }
                }
                return true;
            }
        } // namespace graph
    } // namespace pass

    void ir::Instruction::setGNode(std::shared_ptr<graph::GNode> gnode)
    {
        m_gnode = gnode;
        auto& tag = (*gnode)["Kernel_Selection_Result"];
        if (tag.is_valid())
            m_kernel = tag.as<pass::graph::DefaultKernelSelector::Result>().second;
    }

    std::shared_ptr<TranslationUnit> visit_graph(std::shared_ptr<graph::Graph> graph)
    {
        auto tu = std::make_shared<TranslationUnit>();
        tu->m_graph = graph;
        auto bb = std::make_shared<ir::BasicBlock>();
        for (auto& node : graph->get_ordered_ops())
        {
            auto ins = std::make_shared<ir::Instruction>();
            ins->setGNode(node);
            bb->push_back(ins);
            if (node->is_parameter())
                tu->arg.push_back(node->get_output_tensor_ptr(0));
        }
        for (auto& node : graph->get_outputs())
            tu->out.push_back(node->get_output_tensor_ptr(0));
        tu->program.push_back(bb);
        return tu;
    }
} // namespace nnfusion
