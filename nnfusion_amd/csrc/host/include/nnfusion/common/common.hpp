// Common vocabulary of the host side: device types, shapes, string helpers, checks and logging.
// The class, enum and macro names follow microsoft/nnfusion (src/nnfusion/common/*.hpp,
// src/nnfusion/util/{errors,logging}.hpp) so that a kernel emitter written against that tree
// compiles against this one; the implementations are independent.
#pragma once

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <functional>
#include <iostream>
#include <map>
#include <memory>
#include <set>
#include <sstream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <utility>
#include <vector>

// nnfusion sources use the standard names unqualified
using namespace std;

namespace nnfusion
{
    // src/nnfusion/common/device_type.hpp:10-21
    enum NNFusion_DeviceType
    {
        CUDA_GPU,
        ROCM_GPU,
        GENERIC_CPU,
        HLSL,
        GraphCore,
        UNKNOWN
    };

    inline std::string get_device_str(NNFusion_DeviceType dt)
    {
        switch (dt)
        {
        case CUDA_GPU: return "CUDA_GPU";
        case ROCM_GPU: return "ROCM_GPU";
        case GENERIC_CPU: return "GENERIC_CPU";
        case HLSL: return "HLSL";
        case GraphCore: return "GraphCore";
        default: return "UNKNOWN";
        }
    }

    inline NNFusion_DeviceType get_device_type(const std::string& s)
    {
        if (s == "CUDA" || s == "CUDA_GPU") return CUDA_GPU;
        if (s == "ROCm" || s == "ROCM" || s == "ROCM_GPU") return ROCM_GPU;
        if (s == "CPU" || s == "GENERIC_CPU") return GENERIC_CPU;
        if (s == "HLSL") return HLSL;
        if (s == "GraphCore") return GraphCore;
        return UNKNOWN;
    }

    // ---- shapes -------------------------------------------------------------------------------
    class Shape : public std::vector<size_t>
    {
    public:
        using std::vector<size_t>::vector;
        Shape() = default;
        Shape(const std::vector<size_t>& v)
            : std::vector<size_t>(v)
        {
        }
    };
    using PartialShape = Shape;
    using AxisSet = std::set<size_t>;

    inline size_t shape_size(const Shape& shape)
    {
        size_t n = 1;
        for (size_t d : shape)
            n *= d;
        return n;
    }

    template <typename Container>
    std::string join(const Container& c, const std::string& sep = ", ")
    {
        std::ostringstream ss;
        bool first = true;
        for (const auto& v : c)
        {
            if (!first)
                ss << sep;
            ss << v;
            first = false;
        }
        return ss.str();
    }

    inline std::ostream& operator<<(std::ostream& os, const Shape& s)
    {
        return os << "Shape{" << join(s) << "}";
    }

    // ---- checks: NNFUSION_CHECK(cond) << "message";  throws nnfusion::CheckError when cond is false
    class CheckError : public std::runtime_error
    {
    public:
        explicit CheckError(const std::string& what)
            : std::runtime_error(what)
        {
        }
    };

    namespace detail
    {
        class CheckStream
        {
        public:
            CheckStream(const char* file, int line, const char* expr)
            {
                m_ss << "Check failed: '" << expr << "' at " << file << ":" << line << ": ";
            }
            [[noreturn]] ~CheckStream() noexcept(false) { throw CheckError(m_ss.str()); }
            template <typename T>
            CheckStream& operator<<(const T& v)
            {
                m_ss << v;
                return *this;
            }

        private:
            std::ostringstream m_ss;
        };

        struct Voidify
        {
            void operator&(const CheckStream&) {}
        };

        class LogStream
        {
        public:
            LogStream(int level, const char* tag)
                : m_level(level)
            {
                m_ss << "[" << tag << "] ";
            }
            ~LogStream();
            template <typename T>
            LogStream& operator<<(const T& v)
            {
                m_ss << v;
                return *this;
            }

        private:
            int m_level;
            std::ostringstream m_ss;
        };
    } // namespace detail

    // 0 DEBUG, 1 INFO, 2 WARNING, 3 ERROR; messages below the threshold are dropped
    int& min_log_level();
} // namespace nnfusion

#define NNFUSION_CHECK(cond)                                                                                   \
    (cond) ? (void)0 : ::nnfusion::detail::Voidify() & ::nnfusion::detail::CheckStream(__FILE__, __LINE__, #cond)
#define NNFUSION_CHECK_NOT_NULLPTR(p) NNFUSION_CHECK((p) != nullptr)
#define NNFUSION_CHECK_FAIL() ::nnfusion::detail::CheckStream(__FILE__, __LINE__, "unconditional failure")
#define OP_VALIDATION(op, cond) NNFUSION_CHECK(cond) << "while validating op " << (op)->get_op_type() << ": "

#define NNFUSION_LOG_DEBUG ::nnfusion::detail::LogStream(0, "DEBUG")
#define NNFUSION_LOG_INFO ::nnfusion::detail::LogStream(1, "INFO")
#define NNFUSION_LOG_NNFUSION_WARNING ::nnfusion::detail::LogStream(2, "WARNING")
#define NNFUSION_LOG_ERROR ::nnfusion::detail::LogStream(3, "ERROR")
#define NNFUSION_LOG(level) NNFUSION_LOG_##level
