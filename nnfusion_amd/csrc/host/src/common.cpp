// Logging, element types, CodeWriter / LanguageUnit / FunctionUnit, json_lite.
#include "nnfusion/common/common.hpp"
#include "nnfusion/common/json_lite.hpp"
#include "nnfusion/common/languageunit.hpp"
#include "nnfusion/common/type/element_type.hpp"

#include <cctype>
#include <cerrno>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sys/stat.h>

namespace nnfusion
{
    int& min_log_level()
    {
        static int level = []() {
            const char* e = std::getenv("NNFUSION_MIN_LOG_LEVEL");
            return e ? std::atoi(e) : 2; // warnings and errors unless asked otherwise
        }();
        return level;
    }

    detail::LogStream::~LogStream()
    {
        if (m_level >= min_log_level())
            std::cerr << m_ss.str() << std::endl;
    }

    namespace element
    {
        const Type dynamic(0, false, false, false, "dynamic");
        const Type boolean(8, false, true, false, "char");
        const Type character(8, false, false, false, "char");
        const Type bf16(16, true, true, false, "bfloat16");
        const Type f16(16, true, true, false, "half");
        const Type f32(32, true, true, false, "float");
        const Type f64(64, true, true, false, "double");
        const Type i8(8, false, true, true, "int8_t");
        const Type i16(16, false, true, false, "int16_t");
        const Type i32(32, false, true, true, "int32_t");
        const Type i64(64, false, true, false, "int64_t");
        const Type u8(8, false, false, true, "uint8_t");
        const Type u16(16, false, false, false, "uint16_t");
        const Type u32(32, false, false, false, "uint32_t");
        const Type u64(64, false, false, false, "uint64_t");

        template <> const Type& from<float>() { return f32; }
        template <> const Type& from<double>() { return f64; }
        template <> const Type& from<int8_t>() { return i8; }
        template <> const Type& from<uint8_t>() { return u8; }
        template <> const Type& from<int32_t>() { return i32; }
        template <> const Type& from<int64_t>() { return i64; }
    } // namespace element

    // ---- CodeWriter ----------------------------------------------------------------------------
    void codegen::CodeWriter::write(const std::string& s)
    {
        for (char c : s)
        {
            if (c == '\n')
            {
                m_ss << c;
                m_pending_indent = true;
            }
            else
            {
                if (m_pending_indent)
                {
                    for (size_t i = 0; i < indent; ++i)
                        m_ss << "    ";
                    m_pending_indent = false;
                }
                m_ss << c;
            }
        }
    }

    // ---- LanguageUnit --------------------------------------------------------------------------
    bool LanguageUnit::require(std::shared_ptr<LanguageUnit> lu)
    {
        if (!lu)
            return false;
        NNFUSION_CHECK(lu.get() != this) << "a language unit cannot require itself: " << symbol;
        required.insert(lu->symbol);
        local_symbol[lu->symbol] = lu;
        return true;
    }

    bool LanguageUnit::remove(std::shared_ptr<LanguageUnit> lu)
    {
        if (!lu)
            return false;
        required.erase(lu->symbol);
        return local_symbol.erase(lu->symbol) > 0;
    }

    bool LanguageUnit::replace(std::shared_ptr<LanguageUnit> a, std::shared_ptr<LanguageUnit> b)
    {
        return remove(a) && require(b);
    }

    namespace
    {
        // rank of a symbol in the written file: headers, then macros, then declarations, then the rest
        int symbol_rank(const std::string& sym)
        {
            if (sym.rfind("header::", 0) == 0) return 0;
            if (sym.rfind("macro::", 0) == 0) return 1;
            if (sym.rfind("declaration::", 0) == 0) return 2;
            return 3;
        }

        void collect(LanguageUnit* lu, std::vector<LanguageUnit*>& order, std::unordered_set<std::string>& seen)
        {
            // dependencies first; among the dependencies of one unit, by rank then by symbol (deterministic)
            std::vector<LanguageUnit*> deps;
            for (auto& kv : lu->local_symbol)
                deps.push_back(kv.second.get());
            std::sort(deps.begin(), deps.end(), [](LanguageUnit* x, LanguageUnit* y) {
                int rx = symbol_rank(x->symbol), ry = symbol_rank(y->symbol);
                return rx != ry ? rx < ry : x->symbol < y->symbol;
            });
            for (auto* d : deps)
                if (!seen.count(d->symbol))
                    collect(d, order, seen);
            if (seen.insert(lu->symbol).second)
                order.push_back(lu);
        }
    } // namespace

    std::string LanguageUnit::collect_required_code()
    {
        std::vector<LanguageUnit*> order;
        std::unordered_set<std::string> seen;
        collect(this, order, seen);
        std::stable_sort(order.begin(), order.end() - 1, [](LanguageUnit* x, LanguageUnit* y) {
            return symbol_rank(x->symbol) < symbol_rank(y->symbol);
        });
        std::string code;
        for (size_t i = 0; i + 1 < order.size(); ++i)
            code += order[i]->get_code();
        return code;
    }

    std::string LanguageUnit::collect_code() { return collect_required_code() + get_code(); }

    namespace
    {
        bool make_dirs(const std::string& path)
        {
            std::string cur;
            for (size_t i = 0; i < path.size(); ++i)
            {
                cur += path[i];
                if (path[i] == '/' || i + 1 == path.size())
                {
                    if (cur == "/" || cur == "./" || cur == ".")
                        continue;
                    if (mkdir(cur.c_str(), 0755) != 0 && errno != EEXIST)
                        return false;
                }
            }
            return true;
        }
    } // namespace

    void LanguageUnit::execute(bool append)
    {
        if (write_to.empty())
            return;
        std::string dir = pwd.empty() ? "./" : pwd;
        if (dir.back() != '/')
            dir += '/';
        NNFUSION_CHECK(make_dirs(dir)) << "cannot create " << dir;
        std::ofstream f(dir + write_to, append ? std::ios::app : std::ios::trunc);
        NNFUSION_CHECK(f.good()) << "cannot write " << dir + write_to;
        f << get_code();
    }

    std::string FunctionUnit::get_specialized_signature(std::string func_name)
    {
        NNFUSION_CHECK_NOT_NULLPTR(name_unit);
        NNFUSION_CHECK_NOT_NULLPTR(signature_unit);
        std::string fname = func_name.empty() ? name_unit->get_code() : func_name;
        std::string sig = signature_unit->get_code();
        size_t pos = sig.find_last_of('(');
        NNFUSION_CHECK(pos != std::string::npos && pos > 0) << "signature without '(': " << sig;
        return sig.substr(0, pos) + fname + sig.substr(pos);
    }

    std::string FunctionUnit::get_specialized_function_call(std::string func_name)
    {
        NNFUSION_CHECK_NOT_NULLPTR(name_unit);
        NNFUSION_CHECK_NOT_NULLPTR(call_unit);
        return (func_name.empty() ? name_unit->get_code() : func_name) + call_unit->get_code();
    }

    // ---- json_lite -----------------------------------------------------------------------------
    std::string json_lite::dump() const
    {
        std::ostringstream ss;
        switch (m_kind)
        {
        case Null: ss << "null"; break;
        case Bool: ss << (m_i ? "true" : "false"); break;
        case Int: ss << m_i; break;
        case Float: ss << m_f; break;
        case String: ss << '"' << m_s << '"'; break;
        case Array:
        {
            ss << '[';
            for (size_t i = 0; i < m_a.size(); ++i)
                ss << (i ? "," : "") << m_a[i].dump();
            ss << ']';
            break;
        }
        case Object:
        {
            ss << '{';
            bool first = true;
            for (auto& kv : m_o)
            {
                ss << (first ? "" : ",") << '"' << kv.first << "\":" << kv.second.dump();
                first = false;
            }
            ss << '}';
            break;
        }
        }
        return ss.str();
    }

    namespace
    {
        struct Parser
        {
            const std::string& s;
            size_t p = 0;
            void ws()
            {
                while (p < s.size() && std::isspace((unsigned char)s[p]))
                    ++p;
            }
            json_lite value()
            {
                ws();
                NNFUSION_CHECK(p < s.size()) << "json_lite: unexpected end of text";
                char c = s[p];
                if (c == '{')
                {
                    json_lite obj = json_lite::object();
                    ++p;
                    ws();
                    while (p < s.size() && s[p] != '}')
                    {
                        ws();
                        NNFUSION_CHECK(s[p] == '"') << "json_lite: expected a key at " << p;
                        std::string key = str();
                        ws();
                        NNFUSION_CHECK(p < s.size() && s[p] == ':') << "json_lite: expected ':'";
                        ++p;
                        obj[key] = value();
                        ws();
                        if (p < s.size() && s[p] == ',')
                            ++p;
                        ws();
                    }
                    NNFUSION_CHECK(p < s.size()) << "json_lite: unterminated object";
                    ++p;
                    return obj;
                }
                if (c == '[')
                {
                    json_lite arr = json_lite::array();
                    ++p;
                    ws();
                    while (p < s.size() && s[p] != ']')
                    {
                        arr.push_back(value());
                        ws();
                        if (p < s.size() && s[p] == ',')
                            ++p;
                        ws();
                    }
                    NNFUSION_CHECK(p < s.size()) << "json_lite: unterminated array";
                    ++p;
                    return arr;
                }
                if (c == '"')
                    return json_lite(str());
                if (s.compare(p, 4, "true") == 0)
                {
                    p += 4;
                    return json_lite(true);
                }
                if (s.compare(p, 5, "false") == 0)
                {
                    p += 5;
                    return json_lite(false);
                }
                if (s.compare(p, 4, "null") == 0)
                {
                    p += 4;
                    return json_lite();
                }
                size_t start = p;
                bool is_float = false;
                while (p < s.size() && (std::isdigit((unsigned char)s[p]) || s[p] == '-' || s[p] == '+' || s[p] == '.' ||
                                        s[p] == 'e' || s[p] == 'E'))
                {
                    if (s[p] == '.' || s[p] == 'e' || s[p] == 'E')
                        is_float = true;
                    ++p;
                }
                NNFUSION_CHECK(p > start) << "json_lite: unexpected character '" << c << "' at " << start;
                std::string num = s.substr(start, p - start);
                if (is_float)
                    return json_lite(std::strtod(num.c_str(), nullptr));
                return json_lite((long long)std::strtoll(num.c_str(), nullptr, 10));
            }
            std::string str()
            {
                ++p; // opening quote
                std::string out;
                while (p < s.size() && s[p] != '"')
                {
                    if (s[p] == '\\' && p + 1 < s.size())
                        ++p;
                    out += s[p++];
                }
                NNFUSION_CHECK(p < s.size()) << "json_lite: unterminated string";
                ++p;
                return out;
            }
        };
    } // namespace

    json_lite json_lite::parse(const std::string& text)
    {
        Parser ps{text};
        json_lite v = ps.value();
        ps.ws();
        NNFUSION_CHECK(ps.p == text.size()) << "json_lite: trailing characters";
        return v;
    }
} // namespace nnfusion
