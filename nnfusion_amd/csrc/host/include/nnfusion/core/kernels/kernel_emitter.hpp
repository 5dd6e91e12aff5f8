// KernelContext / KernelEmitter: the kernel plugin API
// (src/nnfusion/core/kernels/kernel_emitter.hpp:18-160, kernel_emitter.cpp:14-48,50-399).
// An emitter turns a graph node into a FunctionUnit (name, signature, body, dependencies, call,
// comments); returning nullptr from emit_function_body() declines the node.
#pragma once

#include "nnfusion/common/descriptor/tensor.hpp"
#include "nnfusion/common/json_lite.hpp"
#include "nnfusion/common/languageunit.hpp"
#include "nnfusion/core/graph/gnode.hpp"

namespace nnfusion
{
    namespace kernels
    {
        class KernelEmitter;

        class KernelContext
        {
        public:
            using Pointer = std::shared_ptr<KernelContext>;
            explicit KernelContext(std::shared_ptr<graph::GNode> gnode);
            KernelContext() = default;
            // op type + shapes + dtypes: identical nodes give identical identifiers
            std::string generate_identifier();

            std::shared_ptr<graph::GNode> gnode;
            std::shared_ptr<op::Op> op;
            std::vector<std::shared_ptr<descriptor::Tensor>> inputs, outputs, tensors;
            std::vector<std::string> input_names, output_names, tensor_names;
            std::vector<std::string> dtypes; // C type strings of inputs then outputs
            uint32_t gpu_num_sm = 20;        // the reference hard-codes 20; emitters here do not use it
            std::vector<std::shared_ptr<KernelEmitter>> kernels;
            std::shared_ptr<Annotations> annotations;
        };

        class KernelEmitter
        {
        public:
            using Pointer = std::shared_ptr<KernelEmitter>;
            explicit KernelEmitter(std::shared_ptr<KernelContext> ctx);
            KernelEmitter(std::shared_ptr<KernelContext> ctx, const std::string& kernel_type);
            virtual ~KernelEmitter() = default;

            // Emits once; with emit_func_call = true an already emitted kernel re-emits only its call unit
            // (stream assignment may change between selection and codegen).
            virtual FunctionUnit_p get_or_emit_source(bool emit_func_call = false);
            virtual FunctionUnit_p emit_source();

            std::string get_kernel_type() { return m_kernel_type; }
            std::string get_function_name() { return m_kernel_name; }
            bool is_emitted() { return m_is_emitted; }
            virtual bool is_static_function() { return false; }
            virtual bool is_parallelism() { return m_intra_op_parallelism; }
            virtual bool is_eliminative() { return false; }
            bool is_tuned() { return m_is_tuned; }
            // "cuda"/"cuda_lib" -> CUDA_GPU, "cpu" -> GENERIC_CPU, "hlsl", "rocm" -> ROCM_GPU, "graphcore"
            NNFusion_DeviceType get_device_type();

            std::shared_ptr<KernelContext> m_context;

        protected:
            // <OpType>_<dtype0>_<dtype1>..._<kernel_type>_<op unique name>
            virtual LanguageUnit_p emit_function_name();
            virtual LanguageUnit_p emit_function_body() = 0;
            // "void (T0* input0, ..., Tk* output0, ..., Ts* scratch...)"
            virtual LanguageUnit_p emit_function_signature();
            virtual LanguageUnit_p emit_dependency() = 0;
            // "(<input names>, <output names>, <scratch names>);\n", the stream name first when the
            // signature text asks for one
            virtual LanguageUnit_p emit_function_call();
            virtual LanguageUnit_p emit_comments();
            // a scratch / persistent tensor owned by this kernel; appended to m_context->tensors and to
            // the signature and call
            virtual const std::shared_ptr<descriptor::Tensor>
                allocate_tensor(Shape shape, element::Type elt = element::f32, std::string name = "",
                                NNFusion_DeviceType device_type = UNKNOWN, bool is_persistent = false,
                                bool is_constant = false, bool is_parameter = false, bool is_RDMA_tensor = false,
                                const std::string& group = "", int device_id = -1);

            bool m_is_emitted = false;
            const std::string m_kernel_type;
            std::string m_kernel_name;
            std::string custom_tag;
            std::unordered_map<std::string, std::shared_ptr<FunctionUnit>> kernel_definitions;
            nlohmann::json attr;
            FunctionUnit_p m_function_unit;
            bool m_intra_op_parallelism = false;
            bool m_is_tuned = false;
        };
    } // namespace kernels
} // namespace nnfusion
