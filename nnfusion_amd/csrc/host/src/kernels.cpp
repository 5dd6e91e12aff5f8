// KernelContext, KernelEmitter, KernelRegistration / KernelRegistry, the HIP emitter base and the
// language units generated code depends on.
#include "nnfusion/core/kernels/hip_gpu/hip_emitter.hpp"
#include "nnfusion/core/kernels/kernel_registration.hpp"

namespace nnfusion
{
    namespace kernels
    {
        // ---- KernelContext ----------------------------------------------------------------------
        KernelContext::KernelContext(std::shared_ptr<graph::GNode> node)
            : gnode(node)
            , op(node->get_op_ptr())
        {
            for (size_t i = 0; i < node->get_input_size(); ++i)
            {
                auto t = node->get_input_tensor_ptr(i);
                NNFUSION_CHECK_NOT_NULLPTR(t);
                inputs.push_back(t);
                input_names.push_back(t->get_name());
            }
            for (size_t i = 0; i < node->get_output_size(); ++i)
            {
                auto t = node->get_output_tensor_ptr(i);
                NNFUSION_CHECK_NOT_NULLPTR(t);
                outputs.push_back(t);
                output_names.push_back(t->get_name());
            }
            for (auto& t : inputs)
                dtypes.push_back(t->get_element_type().c_type_string());
            for (auto& t : outputs)
                dtypes.push_back(t->get_element_type().c_type_string());
            annotations = op->get_op_annotations();
        }

        std::string KernelContext::generate_identifier()
        {
            std::ostringstream id;
            id << gnode->get_op_type();
            for (auto& t : inputs)
                id << "_i" << join(t->get_shape(), "x");
            for (auto& t : outputs)
                id << "_o" << join(t->get_shape(), "x");
            id << "_" << join(dtypes, "_");
            return id.str();
        }

        // ---- KernelEmitter ----------------------------------------------------------------------
        KernelEmitter::KernelEmitter(std::shared_ptr<KernelContext> ctx)
            : m_context(ctx)
        {
        }

        KernelEmitter::KernelEmitter(std::shared_ptr<KernelContext> ctx, const std::string& kernel_type)
            : m_context(ctx)
            , m_kernel_type(kernel_type)
        {
        }

        NNFusion_DeviceType KernelEmitter::get_device_type()
        {
            static const std::map<std::string, NNFusion_DeviceType> by_type = {
                {"cuda", CUDA_GPU}, {"cuda_lib", CUDA_GPU}, {"cpu", GENERIC_CPU},
                {"hlsl", HLSL},     {"rocm", ROCM_GPU},     {"graphcore", GraphCore}};
            auto it = by_type.find(m_kernel_type);
            return it == by_type.end() ? UNKNOWN : it->second;
        }

        LanguageUnit_p KernelEmitter::emit_function_name()
        {
            LanguageUnit_p lu(new LanguageUnit("function_name"));
            *lu << m_context->gnode->get_op_type() << "_" << join(m_context->dtypes, "_") << "_" << m_kernel_type
                << "_" << m_context->gnode->get_op_ptr()->get_unique_name();
            return lu;
        }

        LanguageUnit_p KernelEmitter::emit_function_signature()
        {
            LanguageUnit_p lu(new LanguageUnit(m_kernel_name + "_sig"));
            std::vector<std::string> params;
            for (size_t i = 0; i < m_context->inputs.size(); ++i)
                params.push_back(m_context->inputs[i]->get_element_type().c_type_string() + "* input" + std::to_string(i));
            for (size_t i = 0; i < m_context->outputs.size(); ++i)
                params.push_back(m_context->outputs[i]->get_element_type().c_type_string() + "* output" + std::to_string(i));
            for (auto& t : m_context->tensors)
                params.push_back(t->get_element_type().c_type_string() + "* " + t->get_name());
            *lu << "void (" << join(params, ", ") << ")";
            return lu;
        }

        LanguageUnit_p KernelEmitter::emit_function_call()
        {
            LanguageUnit_p lu(new LanguageUnit(m_kernel_name + "_call"));
            std::vector<std::string> names;
            // A signature that takes a stream gets the node's stream first (the reference looks for the
            // literal "cudaStream_t", kernel_emitter.cpp:160-181; here the token is hipStream_t).
            if (m_function_unit && m_function_unit->signature_unit &&
                m_function_unit->signature_unit->get_code().find("hipStream_t") != std::string::npos)
            {
                std::string stream = "0";
                auto gnode = m_context->gnode;
                if (gnode && (*gnode)["Async_info_stream"].is_valid())
                    stream = (*gnode)["Async_info_stream"].as<std::string>();
                names.push_back(stream);
            }
            names.insert(names.end(), m_context->input_names.begin(), m_context->input_names.end());
            names.insert(names.end(), m_context->output_names.begin(), m_context->output_names.end());
            names.insert(names.end(), m_context->tensor_names.begin(), m_context->tensor_names.end());
            *lu << "(" << join(names, ", ") << ");\n";
            return lu;
        }

        LanguageUnit_p KernelEmitter::emit_comments()
        {
            LanguageUnit_p lu(new LanguageUnit(m_kernel_name + "_comments"));
            auto describe = [&](const std::shared_ptr<descriptor::Tensor>& t) {
                *lu << "//\t- name: " << t->get_name() << "\ttype: " << t->get_element_type().c_type_string()
                    << "\tshape: " << t->get_shape() << "\n";
            };
            *lu << "// Node name:\t" << m_context->gnode->get_op_ptr()->get_unique_name() << "\n";
            *lu << "// Description:\t" << m_context->gnode->get_op_type() << "\n";
            *lu << "// Input:\n";
            for (auto& t : m_context->inputs)
                describe(t);
            *lu << "// Output:\n";
            for (auto& t : m_context->outputs)
                describe(t);
            if (!m_context->tensors.empty())
            {
                *lu << "// Other tensors in use:\n";
                for (auto& t : m_context->tensors)
                    describe(t);
            }
            return lu;
        }

        FunctionUnit_p KernelEmitter::get_or_emit_source(bool emit_func_call)
        {
            if (m_is_emitted)
            {
                if (emit_func_call && m_function_unit)
                    m_function_unit->call_unit = emit_function_call();
                return m_function_unit;
            }
            m_function_unit = emit_source();
            m_is_emitted = true;
            return m_function_unit;
        }

        FunctionUnit_p KernelEmitter::emit_source()
        {
            FunctionUnit_p fu(new FunctionUnit());
            if (m_kernel_name.empty())
            {
                fu->name_unit = emit_function_name();
                m_kernel_name = fu->name_unit->get_code();
            }
            else
            {
                fu->name_unit = LanguageUnit_p(new LanguageUnit("function_name", m_kernel_name));
            }
            auto cached = kernel_definitions.find(m_kernel_name);
            if (cached != kernel_definitions.end())
                return cached->second;

            // the body may allocate scratch tensors, which the signature and the call must list
            fu->body_unit = emit_function_body();
            if (!fu->body_unit)
                return nullptr; // the emitter declines this node
            NNFUSION_CHECK_NOT_NULLPTR(fu->signature_unit = emit_function_signature());
            m_function_unit = fu; // emit_function_call() reads the signature through m_function_unit
            NNFUSION_CHECK_NOT_NULLPTR(fu->call_unit = emit_function_call());
            NNFUSION_CHECK_NOT_NULLPTR(fu->dep_unit = emit_dependency());
            NNFUSION_CHECK_NOT_NULLPTR(fu->comment_unit = emit_comments());

            // everything the body or the call requires becomes a dependency of the function;
            // then body -> dep and call -> body, which orders headers before kernels in the file
            for (auto& kv : fu->call_unit->local_symbol)
                fu->dep_unit->require(kv.second);
            for (auto& kv : fu->body_unit->local_symbol)
                fu->dep_unit->require(kv.second);
            fu->call_unit->clean_require();
            fu->body_unit->clean_require();
            NNFUSION_CHECK(fu->body_unit->require(fu->dep_unit));
            NNFUSION_CHECK(fu->call_unit->require(fu->body_unit));
            kernel_definitions[m_kernel_name] = fu;
            return fu;
        }

        const std::shared_ptr<descriptor::Tensor>
            KernelEmitter::allocate_tensor(Shape shape, element::Type elt, std::string name,
                                           NNFusion_DeviceType device_type, bool is_persistent, bool is_constant,
                                           bool is_parameter, bool is_RDMA_tensor, const std::string& group,
                                           int device_id)
        {
            if (name.empty())
                name = m_context->gnode->get_op_ptr()->get_unique_name() + "_workspace" +
                       std::to_string(m_context->tensors.size());
            auto t = std::make_shared<descriptor::Tensor>(elt, shape, name, device_type, is_persistent, is_constant,
                                                          is_parameter, is_RDMA_tensor, group, device_id);
            m_context->tensors.push_back(t);
            m_context->tensor_names.push_back(name);
            return t;
        }

        // ---- registry ---------------------------------------------------------------------------
        const std::shared_ptr<KernelRegistration> KernelRegistration::Build()
        {
            NNFUSION_CHECK(!m_op_name.empty()) << "kernel registration without an op name";
            NNFUSION_CHECK(m_device_type != UNKNOWN) << "kernel registration for " << m_op_name << " without a device";
            NNFUSION_CHECK(m_factory != nullptr) << "kernel registration for " << m_op_name << " without a factory";
            return std::shared_ptr<KernelRegistration>(this);
        }

        KernelRegistration& Name(const std::string op_name) { return *(new KernelRegistration(op_name)); }

        KernelRegistry* KernelRegistry::Global()
        {
            static KernelRegistry* registry = new KernelRegistry();
            return registry;
        }

        bool KernelRegistry::RegisterKernel(const std::string op_name, std::shared_ptr<KernelRegistration> registration)
        {
            m_kernel_registry.insert(std::make_pair(op_name, registration));
            return true;
        }

        std::vector<std::shared_ptr<const KernelRegistration>>
            KernelRegistry::FindKernelRegistrations(const std::string op_name, const NNFusion_DeviceType& device_type,
                                                    const element::Type data_type)
        {
            std::vector<std::shared_ptr<const KernelRegistration>> found;
            auto range = m_kernel_registry.equal_range(op_name);
            for (auto it = range.first; it != range.second; ++it)
                if (it->second->m_device_type == device_type && it->second->m_data_type == data_type)
                    found.push_back(it->second);
            return found;
        }

        std::shared_ptr<const KernelRegistration>
            KernelRegistry::FindKernelRegistration(const std::string op_name, const NNFusion_DeviceType& device_type,
                                                   const element::Type data_type)
        {
            auto found = FindKernelRegistrations(op_name, device_type, data_type);
            return found.empty() ? nullptr : KernelSelect(found);
        }

        std::shared_ptr<const KernelRegistration>
            KernelRegistry::KernelSelect(std::vector<std::shared_ptr<const KernelRegistration>>& matched_regs)
        {
            std::shared_ptr<const KernelRegistration> best;
            for (auto& r : matched_regs)
                if (!best || r->m_priority > best->m_priority)
                    best = r;
            return best;
        }

        // ---- language units of generated HIP host code -----------------------------------------------
        // (defined with qualified names so that the symbol carries the header:: / macro:: / declaration::
        // prefix the code generator orders by)
        LU_DEFINE(header::stdio, "#include <stdio.h>\n")
        LU_DEFINE(header::stdexcept, "#include <stdexcept>\n")
        LU_DEFINE(header::sstream, "#include <sstream>\n")
        LU_DEFINE(header::fstream, "#include <fstream>\n")
        LU_DEFINE(header::vector, "#include <vector>\n")
        LU_DEFINE(header::chrono, "#include <chrono>\n")
        LU_DEFINE(header::hip, "#include <hip/hip_runtime.h>\n")
        LU_DEFINE(header::nnf_hip_kernels, "#include \"nnf_hip_kernels.h\"\n")
        LU_DEFINE(macro::HIP_SAFE_CALL,
                      R"(#define HIP_SAFE_CALL(x)                                                                   \
    do                                                                                                \
    {                                                                                                 \
        hipError_t result = (x);                                                                      \
        if (result != hipSuccess)                                                                     \
        {                                                                                             \
            std::stringstream safe_call_ss;                                                           \
            safe_call_ss << "\nerror: " #x " failed with error"                                       \
                         << "\nfile: " << __FILE__ << "\nline: " << __LINE__                          \
                         << "\nmsg: " << hipGetErrorString(result);                                   \
            throw std::runtime_error(safe_call_ss.str());                                             \
        }                                                                                             \
    } while (0)
)")
        LU_DEFINE(macro::NNF_HIP_CHECK,
                      R"(#define NNF_HIP_CHECK(x)                                                                   \
    do                                                                                                \
    {                                                                                                 \
        int nnf_status = (x);                                                                         \
        if (nnf_status != 0)                                                                          \
        {                                                                                             \
            std::stringstream safe_call_ss;                                                           \
            safe_call_ss << "\nerror: " #x " failed with status " << nnf_status                       \
                         << "\nfile: " << __FILE__ << "\nline: " << __LINE__                          \
                         << "\nmsg: " << nnf_status_string(nnf_status);                               \
            throw std::runtime_error(safe_call_ss.str());                                             \
        }                                                                                             \
    } while (0)
)")
        LU_DEFINE(declaration::typedef_half, "typedef _Float16 half;\n")
        LU_DEFINE(declaration::typedef_int, "#include <stdint.h>\n#include <stddef.h>\n")

        // ---- HipLibEmitter ------------------------------------------------------------------------
        LanguageUnit_p hip::HipLibEmitter::emit_function_signature()
        {
            LanguageUnit_p lu(new LanguageUnit(m_kernel_name + "_sig"));
            std::vector<std::string> params{"hipStream_t stream"};
            for (size_t i = 0; i < m_context->inputs.size(); ++i)
                params.push_back(m_context->inputs[i]->get_element_type().c_type_string() + "* input" + std::to_string(i));
            for (size_t i = 0; i < m_context->outputs.size(); ++i)
                params.push_back(m_context->outputs[i]->get_element_type().c_type_string() + "* output" + std::to_string(i));
            for (auto& t : m_context->tensors)
                params.push_back(t->get_element_type().c_type_string() + "* " + t->get_name());
            *lu << "void (" << join(params, ", ") << ")";
            return lu;
        }

        LanguageUnit_p hip::HipLibEmitter::emit_dependency()
        {
            LanguageUnit_p lu(new LanguageUnit(get_function_name() + "_dep"));
            lu->require(header::hip);
            lu->require(header::stdexcept);
            lu->require(header::sstream);
            lu->require(header::nnf_hip_kernels);
            lu->require(macro::NNF_HIP_CHECK);
            lu->require(declaration::typedef_int);
            lu->require(declaration::typedef_half);
            return lu;
        }
    } // namespace kernels
} // namespace nnfusion
