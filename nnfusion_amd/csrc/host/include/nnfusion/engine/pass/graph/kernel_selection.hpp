// DefaultKernelSelector: picks, per node, the first registered emitter (by priority) that emits
// (src/nnfusion/engine/pass/graph/kernel_selection.cpp:139-299), and DefaultGNodeDeviceDispatcher, which
// tags every node with the default device (gnode_device_dispatcher.cpp:12-94).
#pragma once

#include "nnfusion/core/kernels/kernel_registration.hpp"
#include "nnfusion/engine/profiler/hip_runtime.hpp"

#include <map>

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

            // ProfilingBasedKernelSelector (src/nnfusion/engine/pass/graph/kernel_selection.cpp:21-137): for the
            // operators of a white list, every registered emitter that accepts the node is run through the
            // single-kernel harness and the fastest is stored as "Kernel_Selection_Result", which
            // DefaultKernelSelector then keeps.  The reference's white list is {"Broadcast"}; here it is
            // {"QuantDot"}, whose emitters are the automatic one and the four kernel variants.
            class ProfilingBasedKernelSelector
            {
            public:
                using Result = DefaultKernelSelector::Result;
                struct Timing
                {
                    std::string kernel_type;
                    double ms; // mean of runtime_times runs; < 0: failed to compile or run
                };
                bool enable = true; // the reference's -fkernel_selection
                // only generate and compile the harnesses (a host without the device): nothing runs, nothing is chosen;
                // a later run with the same working_dir finds the objects and compiles nothing
                bool prepare_only = false;
                size_t warmup_times = 5, runtime_times = 100;
                std::string working_dir = "./kernel_profiling/";

                // every registered emitter of the node's operator (ROCM_GPU: CUDA_GPU registrations too) that emits for it
                std::vector<kernels::KernelEmitter::Pointer> candidates(std::shared_ptr<nnfusion::graph::GNode> gnode,
                                                                        NNFusion_DeviceType devtype);
                // harness contexts of the candidates, sources generated (no compiler, no device)
                std::vector<profiler::ProfilingContext::Pointer> contexts(std::shared_ptr<nnfusion::graph::GNode> gnode,
                                                                          NNFusion_DeviceType devtype,
                                                                          profiler::HipDefaultRuntime& runtime);
                // Compiles and runs every candidate on deterministic pseudo-random inputs; second == nullptr if
                // fewer than two candidates exist (nothing to choose) or none ran.  timings (optional): one entry
                // per candidate; outputs (optional): the first output blob of every candidate that ran.
                Result profiling_best(std::shared_ptr<nnfusion::graph::GNode> gnode, NNFusion_DeviceType devtype,
                                      profiler::HipDefaultRuntime& runtime, std::vector<Timing>* timings = nullptr,
                                      std::vector<std::vector<uint8_t>>* outputs = nullptr);
                // nodes of equal identifier (operator, shapes, types) are profiled once
                bool run_on_graph(std::shared_ptr<nnfusion::graph::Graph>& graph, profiler::HipDefaultRuntime& runtime);

            private:
                std::map<std::string, std::string> m_best_type; // identifier -> kernel type of the winner
            };
        } // namespace graph
    } // namespace pass
} // namespace nnfusion
