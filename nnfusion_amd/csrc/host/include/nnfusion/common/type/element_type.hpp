// element::Type: the element types a tensor can carry (src/nnfusion/common/type/element_type.hpp:41-119,
// .cpp:24-38 in the nnfusion tree).  There is no 4-bit type: int4 weights travel as u8 [N, K/2].
#pragma once

#include "nnfusion/common/common.hpp"

namespace nnfusion
{
    namespace element
    {
        class Type
        {
        public:
            Type() = default;
            Type(size_t bitwidth, bool is_real, bool is_signed, bool is_quantized, const std::string& cname)
                : m_bitwidth(bitwidth)
                , m_is_real(is_real)
                , m_is_signed(is_signed)
                , m_is_quantized(is_quantized)
                , m_cname(cname)
            {
            }
            const std::string& c_type_string() const { return m_cname; }
            size_t size() const { return (m_bitwidth + 7) / 8; }
            size_t bitwidth() const { return m_bitwidth; }
            bool is_real() const { return m_is_real; }
            bool is_signed() const { return m_is_signed; }
            bool is_quantized() const { return m_is_quantized; }
            bool operator==(const Type& o) const
            {
                return m_bitwidth == o.m_bitwidth && m_is_real == o.m_is_real && m_is_signed == o.m_is_signed &&
                       m_is_quantized == o.m_is_quantized && m_cname == o.m_cname;
            }
            bool operator!=(const Type& o) const { return !(*this == o); }
            bool operator<(const Type& o) const { return m_cname < o.m_cname; }
            // Type::merge: two static types merge only when equal (op::Dot relies on this to reject
            // mixed inputs, src/nnfusion/core/operators/op_define/dot.cpp:47-53)
            static bool merge(Type& dst, const Type& a, const Type& b)
            {
                if (a != b)
                    return false;
                dst = a;
                return true;
            }

        private:
            size_t m_bitwidth = 0;
            bool m_is_real = false, m_is_signed = false, m_is_quantized = false;
            std::string m_cname = "dynamic";
        };

        inline std::ostream& operator<<(std::ostream& os, const Type& t) { return os << "element::Type{" << t.c_type_string() << "}"; }

        extern const Type dynamic, boolean, character, bf16, f16, f32, f64, i8, i16, i32, i64, u8, u16, u32, u64;

        template <typename T>
        const Type& from();
    } // namespace element
} // namespace nnfusion
