// LU_DECLARE / LU_DEFINE: named language units for headers, macros and declarations that kernels
// depend on (src/nnfusion/core/kernels/common_langunit.hpp:7-14).  Symbols start with "header::",
// "macro::" or "declaration::"; the code generator writes them in that order before any kernel.
#pragma once

#include "nnfusion/common/languageunit.hpp"

#define LU_DECLARE(NAME) extern ::nnfusion::LanguageUnit_p NAME;
#define LU_DEFINE(NAME, code) ::nnfusion::LanguageUnit_p NAME = ::nnfusion::LanguageUnit_p(new ::nnfusion::LanguageUnit(#NAME, code));

namespace nnfusion
{
    namespace kernels
    {
        namespace header
        {
            LU_DECLARE(stdio)
            LU_DECLARE(stdexcept)
            LU_DECLARE(sstream)
            LU_DECLARE(fstream)
            LU_DECLARE(vector)
            LU_DECLARE(chrono)
            // <hip/hip_runtime.h> and the C ABI of the gfx950 launcher library
            LU_DECLARE(hip)
            LU_DECLARE(nnf_hip_kernels)
        } // namespace header
        namespace macro
        {
            // HIP_SAFE_CALL(expr): throws std::runtime_error with expression, file and line
            LU_DECLARE(HIP_SAFE_CALL)
            // NNF_HIP_CHECK(status): the same for the launcher library's status codes
            LU_DECLARE(NNF_HIP_CHECK)
        } // namespace macro
        namespace declaration
        {
            // `half` for generated signatures (element::f16's C type string is "half") and the
            // fixed-width integer typedefs
            LU_DECLARE(typedef_half)
            LU_DECLARE(typedef_int)
        } // namespace declaration
    } // namespace kernels
} // namespace nnfusion
