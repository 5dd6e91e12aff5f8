// Single-kernel harness: the protocol the reference's kernel tests use
// (src/nnfusion/engine/profiler/{profiler.hpp:44-239, profiling_runtime.hpp:469-569, cuda_runtime.cpp:18-475,
// rocm_runtime.cpp:15-117}): generate a translation unit around ONE emitted kernel with
//   extern "C" double <name>_entry(void** args, void** outputs)     // host blobs in, host blobs out, mean ms back
// compile it with hipcc into a shared object, dlopen it and call the entry.
#pragma once

#include "nnfusion/core/kernels/kernel_emitter.hpp"

namespace nnfusion
{
    namespace profiler
    {
        struct ProfilingContext
        {
            using Pointer = std::shared_ptr<ProfilingContext>;
            explicit ProfilingContext(kernels::KernelEmitter::Pointer k)
                : kernel(k)
            {
            }
            kernels::KernelEmitter::Pointer kernel;
            size_t warmup_times = 5;
            size_t runtime_times = 100;
            std::string working_dir = "./kernel_profiling/";
            // filled by HipDefaultRuntime
            std::string source_code, source_path, object_path, entry_name;
            void* handle = nullptr;
            double (*entry_point)(void**, void**) = nullptr;
        };

        class HipDefaultRuntime
        {
        public:
            // where nnf_hip_kernels.h and libnnf_hip_kernels.so live
            HipDefaultRuntime(const std::string& include_dir, const std::string& lib_dir)
                : m_include_dir(include_dir)
                , m_lib_dir(lib_dir)
            {
            }
            // hipcc present?
            bool check_env() const;
            // source text of the harness around ke->kernel (no compiler, no device)
            bool codegen(ProfilingContext::Pointer ke);
            // writes the source and compiles it with hipcc --offload-arch=gfx950 -shared
            bool compile(ProfilingContext::Pointer ke);
            // dlopen + one call of <name>_entry; returns mean milliseconds, < 0 on failure
            double execute(ProfilingContext::Pointer ke, void** inputs, void** outputs);

        private:
            std::string m_include_dir, m_lib_dir;
        };
    } // namespace profiler
} // namespace nnfusion
