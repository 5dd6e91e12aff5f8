// A small JSON-like value for operator attributes.  The nnfusion tree uses nlohmann::json for
// OpConfig attributes (src/nnfusion/core/operators/generic_op/generic_op.hpp:54-171); that library is
// not part of this build, so the subset emitters need is provided here: null / bool / integer / float /
// string / array / object, operator[] by key or index, typed get<T>(), dump().
#pragma once

#include "nnfusion/common/common.hpp"

namespace nnfusion
{
    class json_lite
    {
    public:
        enum Kind
        {
            Null,
            Bool,
            Int,
            Float,
            String,
            Array,
            Object
        };
        json_lite() = default;
        json_lite(bool v) : m_kind(Bool), m_i(v) {}
        json_lite(int v) : m_kind(Int), m_i(v) {}
        json_lite(unsigned v) : m_kind(Int), m_i(v) {}
        json_lite(long v) : m_kind(Int), m_i(v) {}
        json_lite(unsigned long v) : m_kind(Int), m_i((int64_t)v) {}
        json_lite(long long v) : m_kind(Int), m_i(v) {}
        json_lite(float v) : m_kind(Float), m_f(v) {}
        json_lite(double v) : m_kind(Float), m_f(v) {}
        json_lite(const char* v) : m_kind(String), m_s(v) {}
        json_lite(const std::string& v) : m_kind(String), m_s(v) {}
        template <typename T>
        json_lite(const std::vector<T>& v) : m_kind(Array)
        {
            for (const auto& e : v)
                m_a.emplace_back(e);
        }

        static json_lite object()
        {
            json_lite v;
            v.m_kind = Object;
            return v;
        }
        static json_lite array()
        {
            json_lite v;
            v.m_kind = Array;
            return v;
        }

        Kind kind() const { return m_kind; }
        bool is_null() const { return m_kind == Null; }
        bool is_number() const { return m_kind == Int || m_kind == Float; }
        bool is_string() const { return m_kind == String; }
        bool is_array() const { return m_kind == Array; }
        bool is_object() const { return m_kind == Object; }
        size_t size() const { return m_kind == Array ? m_a.size() : m_kind == Object ? m_o.size() : 0; }
        bool contains(const std::string& key) const { return m_kind == Object && m_o.count(key); }

        json_lite& operator[](const std::string& key)
        {
            if (m_kind == Null)
                m_kind = Object;
            NNFUSION_CHECK(m_kind == Object) << "json_lite: key access on a non-object";
            return m_o[key];
        }
        const json_lite& at(const std::string& key) const
        {
            auto it = m_o.find(key);
            NNFUSION_CHECK(m_kind == Object && it != m_o.end()) << "json_lite: missing key " << key;
            return it->second;
        }
        json_lite& operator[](size_t i)
        {
            NNFUSION_CHECK(m_kind == Array && i < m_a.size()) << "json_lite: bad index";
            return m_a[i];
        }
        void push_back(const json_lite& v)
        {
            if (m_kind == Null)
                m_kind = Array;
            NNFUSION_CHECK(m_kind == Array);
            m_a.push_back(v);
        }
        const std::map<std::string, json_lite>& items() const { return m_o; }

        template <typename T>
        T get() const;
        template <typename T>
        operator T() const
        {
            return get<T>();
        }
        std::string dump() const;
        // a flat object / scalar parser for per-node configuration strings such as {"group": 128, "zp": 8}
        static json_lite parse(const std::string& text);

    private:
        Kind m_kind = Null;
        int64_t m_i = 0;
        double m_f = 0;
        std::string m_s;
        std::vector<json_lite> m_a;
        std::map<std::string, json_lite> m_o;
        friend struct json_lite_access;
    };

    template <>
    inline bool json_lite::get<bool>() const
    {
        NNFUSION_CHECK(m_kind == Bool || m_kind == Int) << "json_lite: not a bool";
        return m_i != 0;
    }
    template <>
    inline int64_t json_lite::get<int64_t>() const
    {
        NNFUSION_CHECK(is_number() || m_kind == Bool) << "json_lite: not a number";
        return m_kind == Float ? (int64_t)m_f : m_i;
    }
    template <>
    inline int json_lite::get<int>() const { return (int)get<int64_t>(); }
    template <>
    inline size_t json_lite::get<size_t>() const { return (size_t)get<int64_t>(); }
    template <>
    inline double json_lite::get<double>() const
    {
        NNFUSION_CHECK(is_number()) << "json_lite: not a number";
        return m_kind == Float ? m_f : (double)m_i;
    }
    template <>
    inline float json_lite::get<float>() const { return (float)get<double>(); }
    template <>
    inline std::string json_lite::get<std::string>() const
    {
        NNFUSION_CHECK(m_kind == String) << "json_lite: not a string";
        return m_s;
    }
} // namespace nnfusion

// source compatibility for code that spells the attribute type nlohmann::json
namespace nlohmann
{
    using json = ::nnfusion::json_lite;
}
