// DefaultKernelSelector: picks, per node, the first registered emitter (by priority) that emits
// (src/nnfusion/engine/pass/graph/kernel_selection.cpp:139-299), and DefaultGNodeDeviceDispatcher, which
// tags every node with the default device (gnode_device_dispatcher.cpp:12-94).
#pragma once

#include "nnfusion/core/kernels/kernel_registration.hpp"

namespace nnfusion
{
    namespace pass
    {
        namespace graph
        {
            class DefaultGNodeDeviceDispatcher
            {
            public:
                explicit DefaultGNodeDeviceDispatcher(NNFusion_DeviceType dt = ROCM_GPU)
                    : m_device(dt)
                {
                }
                // sets (*gnode)["DeviceType"] and (*gnode)["DeviceID"] on every node
                bool run_on_graph(std::shared_ptr<nnfusion::graph::Graph>& graph);

            private:
                NNFusion_DeviceType m_device;
            };

            class DefaultKernelSelector
            {
            public:
                using Result = std::pair<NNFusion_DeviceType, kernels::KernelEmitter::Pointer>;
                // Lookup key is (op type, devtype, element::f32) whatever the tensor dtypes are; for
                // ROCM_GPU the CUDA_GPU registrations are candidates too; candidates are ordered by
                // priority (+1 when registered for the node's own device), ties by kernel type string;
                // the first whose get_or_emit_source() is non-null wins.  second == nullptr if none emits.
                Result pick_first(std::shared_ptr<nnfusion::graph::GNode> gnode, NNFusion_DeviceType devtype);
                // registers, at priority 10, an emitter around an inline kernel string of the op's OpConfig
                bool register_custom_kernel(const std::string& op_name, NNFusion_DeviceType devtype);
                // stores the winner under the tag "Kernel_Selection_Result"; nodes already tagged are kept
                bool run_on_graph(std::shared_ptr<nnfusion::graph::Graph>& graph);
            };
        } // namespace graph
    } // namespace pass
} // namespace nnfusion
