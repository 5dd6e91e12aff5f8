// GenericOp / OpConfig / REGISTER_OP: how an operator plugin declares a new op
// (src/nnfusion/core/operators/generic_op/generic_op.hpp:13-14,54-171,315-455; custom-op convention in
// src/contrib/custom_op/README.md).  The quantized ops of this build are declared through it
// (src/quant_ops.cpp); they cannot be op::Dot, which rejects mixed input element types.
#pragma once

#include "nnfusion/common/json_lite.hpp"
#include "nnfusion/core/graph/gnode.hpp"

#define REGISTER_OP(op_x)                                                                                      \
    static nnfusion::op::OpConfig& __register_op_##op_x = nnfusion::op::build_op_config(#op_x)

namespace nnfusion
{
    namespace op
    {
        class OpConfig
        {
        public:
            using any = nlohmann::json;
            using constrait_func_t = bool (*)(const OpConfig::any& config);
            using infershape_func_t = void (*)(std::shared_ptr<graph::GNode> gnode);
            using kernel_func_t = std::string (*)(std::shared_ptr<graph::GNode> gnode);

            template <typename T>
            OpConfig& attr(const std::string& name, const T& val = T())
            {
                getRoot()[name] = any(val);
                return *this;
            }
            OpConfig& constrait(const constrait_func_t& func)
            {
                f_constraits.push_back(func);
                return *this;
            }
            OpConfig& infershape(const infershape_func_t& func)
            {
                f_infershape = func;
                return *this;
            }
            // inline kernel source for a device (selected at priority 10 by register_custom_kernel)
            OpConfig& cuda_kernel(const kernel_func_t& func, std::vector<uint32_t> config, bool is_memcpy = false)
            {
                f_kernel_funcs["CUDA_GPU"] = func;
                getRoot()["launch_config"] = any(config);
                getRoot()["is_memcpy"] = any(is_memcpy);
                return *this;
            }
            OpConfig& cpu_kernel(const kernel_func_t& func, bool is_memcpy = false)
            {
                f_kernel_funcs["GENERIC_CPU"] = func;
                getRoot()["is_memcpy"] = any(is_memcpy);
                return *this;
            }
            OpConfig& check_constrait()
            {
                NNFUSION_CHECK(is_legal()) << "OpConfig::check_constrait() not passed!";
                return *this;
            }
            bool is_legal()
            {
                for (auto& f : f_constraits)
                    if (!f(getRoot()))
                        return false;
                return true;
            }
            OpConfig::any& getRoot() { return j_attrs["config"]; }
            OpConfig::any& get(const std::string& key) { return getRoot()[key]; }

            std::vector<constrait_func_t> f_constraits;
            infershape_func_t f_infershape = nullptr;
            std::map<std::string, kernel_func_t> f_kernel_funcs;
            OpConfig::any j_attrs;
        };

        std::unordered_map<std::string, OpConfig>& get_op_configs();
        OpConfig& build_op_config(const std::string& opname);
        OpConfig& lookup_op_config(const std::string& opname);

        // "@key@" substitution used by inline kernels and emitters
        std::string create_code_from_template(std::string templ, const OpConfig::any& feed_dict);

        class GenericOp : public Op
        {
        public:
            // name: instance name; opname: the registered op; customOpConfig: per-node attributes that
            // override the registered defaults
            GenericOp(const std::string& name, const std::string& opname, const OpConfig::any& customOpConfig);
            void validate_and_infer_types(std::shared_ptr<graph::GNode> gnode) override;
            OpConfig localOpConfig;
        };
    } // namespace op
} // namespace nnfusion
