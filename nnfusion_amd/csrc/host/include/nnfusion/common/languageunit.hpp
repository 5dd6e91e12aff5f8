// CodeWriter / LanguageUnit / FunctionUnit: the text containers emitters fill and codegen passes
// consume (src/nnfusion/common/code_writer.hpp, src/nnfusion/common/languageunit.hpp:25-119).
#pragma once

#include "nnfusion/common/common.hpp"

namespace nnfusion
{
    namespace codegen
    {
        // A string stream with block-structured indentation: block_begin() writes "{" and indents,
        // block_end() dedents and writes "}"; every new line gets the current indentation.
        class CodeWriter
        {
        public:
            CodeWriter() = default;
            CodeWriter(const CodeWriter& o)
                : indent(o.indent)
                , m_pending_indent(o.m_pending_indent)
            {
                m_ss << o.m_ss.str();
            }
            CodeWriter& operator=(const CodeWriter& o)
            {
                m_ss.str(o.m_ss.str());
                m_ss.seekp(0, std::ios_base::end);
                indent = o.indent;
                m_pending_indent = o.m_pending_indent;
                return *this;
            }
            template <typename T>
            CodeWriter& operator<<(const T& v)
            {
                std::ostringstream tmp;
                tmp << v;
                write(tmp.str());
                return *this;
            }
            std::string get_code() const { return m_ss.str(); }
            void block_begin()
            {
                *this << "{\n";
                ++indent;
            }
            void block_end()
            {
                --indent;
                *this << "}\n";
            }
            size_t indent = 0;

        protected:
            void write(const std::string& s);
            std::ostringstream m_ss;
            bool m_pending_indent = true;
        };
    } // namespace codegen

    class LanguageUnit : public codegen::CodeWriter
    {
    public:
        std::string symbol;
        std::unordered_set<std::string> required;
        std::unordered_map<std::string, std::shared_ptr<LanguageUnit>> local_symbol;
        std::string pwd;       // directory the unit is written to
        std::string write_to;  // file name inside pwd
        std::vector<std::pair<std::string, std::string>> copy_templates;
        std::vector<std::string> copy_folder;
        std::shared_ptr<LanguageUnit> extern_decl_unit;

        LanguageUnit() = default;
        explicit LanguageUnit(const std::string& sym)
            : symbol(sym)
        {
        }
        LanguageUnit(const std::string& sym, const std::string& code)
            : symbol(sym)
        {
            *this << code;
        }
        virtual ~LanguageUnit() = default;

        bool change_symbol(const std::string& sym)
        {
            symbol = sym;
            return true;
        }
        const std::string& get_symbol() const { return symbol; }
        // by name only (the unit must be supplied later) or by unit
        bool require(const std::string& sym)
        {
            required.insert(sym);
            return true;
        }
        bool require(std::shared_ptr<LanguageUnit> lu);
        bool remove(std::shared_ptr<LanguageUnit> lu);
        bool replace(std::shared_ptr<LanguageUnit> a, std::shared_ptr<LanguageUnit> b);
        void clean_require()
        {
            required.clear();
            local_symbol.clear();
        }
        // code of every (transitively) required unit, dependencies first, each once, then this unit
        std::string collect_code();
        std::string collect_required_code();
        // write collect-free code (this unit only) to pwd/write_to
        virtual void execute(bool append = true);
    };
    using LanguageUnit_p = std::shared_ptr<LanguageUnit>;

    struct FunctionUnit : public LanguageUnit
    {
        LanguageUnit_p name_unit;
        LanguageUnit_p signature_unit; // "void (half* input0, uint8_t* input1, ..., half* output0)"
        LanguageUnit_p body_unit;
        LanguageUnit_p dep_unit;
        LanguageUnit_p call_unit;      // "(tensor_1, tensor_2, tensor_3);\n"
        LanguageUnit_p comment_unit;

        // the signature with the function name spliced in before the last '('
        std::string get_specialized_signature(std::string func_name = "");
        std::string get_specialized_function_call(std::string func_name = "");
    };
    using FunctionUnit_p = std::shared_ptr<FunctionUnit>;
} // namespace nnfusion
