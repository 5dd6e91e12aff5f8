// Base class of the gfx950 emitters: a host function that forwards to the C-ABI launcher library,
// in the place the reference gives to CudaLibEmitter (src/nnfusion/core/kernels/cuda_gpu/cuda_emitter.hpp:190-199:
// a host function around a vendor-library call).  kernel type "rocm" maps to ROCM_GPU.
#pragma once

#include "nnfusion/core/kernels/common_langunit.hpp"
#include "nnfusion/core/kernels/kernel_emitter.hpp"

namespace nnfusion
{
    namespace kernels
    {
        namespace hip
        {
            class HipLibEmitter : public KernelEmitter
            {
            public:
                explicit HipLibEmitter(std::shared_ptr<KernelContext> ctx)
                    : KernelEmitter(ctx, "rocm")
                {
                }
                // kernel_type tells apart several emitters of one operator (it is part of the function name)
                HipLibEmitter(std::shared_ptr<KernelContext> ctx, const std::string& kernel_type)
                    : KernelEmitter(ctx, kernel_type)
                {
                }
                bool is_static_function() override { return false; }

            protected:
                // "void (hipStream_t stream, T0* input0, ..., Tk* output0, ..., Ts* scratch...)"
                LanguageUnit_p emit_function_signature() override;
                // header::hip, header::nnf_hip_kernels, header::stdexcept, macro::NNF_HIP_CHECK, declaration::typedef_half
                LanguageUnit_p emit_dependency() override;
            };
        } // namespace hip
    } // namespace kernels
} // namespace nnfusion
