// CodeGenerator, BaseCodegenPass, HipCodegenPass and the reduced ROCm engine.
//
// The generated project (./nnfusion_rt/rocm_codegen/):
//   nnfusion_rt.h      extern "C" declarations: kernel_entry, rocm_init/rocm_free (and the cuda_init/
//                      cuda_free names the reference's ROCm pass emits, rocm_codegen_pass.cpp:66-68,105),
//                      get_device_type, get_workspace_size
//   nnfusion_rt.cpp    HIP host code: one function per kernel (de-duplicated by signature + body),
//                      init (pool allocation, constants read from Constant/*.bin), kernel_entry, free
//   main_test.cpp      warm-up + timed loop printing "Summary: [min, max, mean]" as the reference's does
//                      (cuda_codegen_pass.cpp:1142-1358)
//   Makefile, CMakeLists.txt, Constant/<tensor>.bin, para_info.json
// It contains no CUDA spelling, needs no hipify step and no CUDA-compat header.
#include "nnfusion/engine/pass/codegen/base_codegen_pass.hpp"
#include "nnfusion/core/kernels/common_langunit.hpp"
#include "nnfusion/engine/pass/graph/kernel_selection.hpp"
#include "nnfusion/engine/pass/graph/quant_fusion_pass.hpp"

#include <cerrno>
#include <cstdlib>
#include <fstream>
#include <sys/stat.h>

namespace nnfusion
{
    namespace codegen
    {
        namespace
        {
            int rank_of(const std::string& sym)
            {
                if (sym.rfind("header::", 0) == 0) return 0;
                if (sym.rfind("macro::", 0) == 0) return 1;
                if (sym.rfind("declaration::", 0) == 0) return 2;
                return 3;
            }

            void gather(LanguageUnit_p lu, std::vector<LanguageUnit_p>& out, std::unordered_set<std::string>& seen)
            {
                std::vector<LanguageUnit_p> deps;
                for (auto& kv : lu->local_symbol)
                    deps.push_back(kv.second);
                std::sort(deps.begin(), deps.end(), [](const LanguageUnit_p& a, const LanguageUnit_p& b) {
                    return a->symbol < b->symbol;
                });
                for (auto& d : deps)
                    if (!seen.count(d->symbol))
                        gather(d, out, seen);
                if (seen.insert(lu->symbol).second)
                    out.push_back(lu);
            }

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

        void CodeGenerator::add(const std::string& file, LanguageUnit_p lu)
        {
            if (!m_files.count(file))
                m_order.push_back(file);
            m_files[file].push_back(lu);
        }

        void CodeGenerator::add_binary(const std::string& file, const void* data, size_t bytes)
        {
            auto& v = m_binaries[file];
            v.assign((const uint8_t*)data, (const uint8_t*)data + bytes);
        }

        std::string CodeGenerator::render(const std::string& file) const
        {
            auto it = m_files.find(file);
            if (it == m_files.end())
                return "";
            // every unit with its transitive requirements, each once; then a stable order:
            // header:: < macro:: < declaration:: < the rest in dependency / insertion order
            std::vector<LanguageUnit_p> all;
            std::unordered_set<std::string> seen;
            for (auto& lu : it->second)
                gather(lu, all, seen);
            std::stable_sort(all.begin(), all.end(), [](const LanguageUnit_p& a, const LanguageUnit_p& b) {
                return rank_of(a->symbol) < rank_of(b->symbol);
            });
            std::string text;
            for (auto& lu : all)
                text += lu->get_code();
            return text;
        }

        std::vector<std::string> CodeGenerator::files() const
        {
            std::vector<std::string> v = m_order;
            for (auto& kv : m_binaries)
                v.push_back(kv.first);
            return v;
        }

        bool CodeGenerator::codegen()
        {
            std::string root = m_codegen_folder;
            if (root.empty())
                root = "./";
            if (root.back() != '/')
                root += '/';
            auto dir_of = [](const std::string& p) {
                size_t pos = p.find_last_of('/');
                return pos == std::string::npos ? std::string() : p.substr(0, pos + 1);
            };
            for (auto& file : m_order)
            {
                if (!make_dirs(root + dir_of(file)))
                    return false;
                std::ofstream f(root + file, std::ios::trunc);
                if (!f.good())
                    return false;
                f << render(file);
            }
            for (auto& kv : m_binaries)
            {
                if (!make_dirs(root + dir_of(kv.first)))
                    return false;
                std::ofstream f(root + kv.first, std::ios::trunc | std::ios::binary);
                if (!f.good())
                    return false;
                f.write((const char*)kv.second.data(), (std::streamsize)kv.second.size());
            }
            return true;
        }

        // ---- BaseCodegenPass -----------------------------------------------------------------------
        bool BaseCodegenPass::run(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu)
        {
            hook_trace.clear();
            initialize(ctx, tu);
            NNFUSION_CHECK(collect_mem(ctx, tu));
            NNFUSION_CHECK(collect_stream(ctx, tu));
            NNFUSION_CHECK(collect_funcs(ctx, tu));
            NNFUSION_CHECK(modify_codegen());
            hook_trace.push_back("codegen");
            NNFUSION_CHECK(projgen->codegen()) << "cannot write below " << m_codegen_folder;
            NNFUSION_CHECK(after_projgen());
            NNFUSION_LOG(INFO) << "Codegen for " << get_device_str(device_type()) << " done.";
            if (exit_after_codegen)
                exit(0);
            return true;
        }

        void BaseCodegenPass::initialize(std::shared_ptr<InterpreterContext>, std::shared_ptr<TranslationUnit>)
        {
            hook_trace.push_back("initialize");
        }
        bool BaseCodegenPass::collect_mem(std::shared_ptr<InterpreterContext>, std::shared_ptr<TranslationUnit>)
        {
            hook_trace.push_back("collect_mem");
            return true;
        }
        bool BaseCodegenPass::collect_stream(std::shared_ptr<InterpreterContext>, std::shared_ptr<TranslationUnit>)
        {
            hook_trace.push_back("collect_stream");
            return true;
        }
        bool BaseCodegenPass::collect_funcs(std::shared_ptr<InterpreterContext>, std::shared_ptr<TranslationUnit>)
        {
            hook_trace.push_back("collect_funcs");
            return true;
        }
        bool BaseCodegenPass::modify_codegen()
        {
            hook_trace.push_back("modify_codegen");
            return true;
        }
        bool BaseCodegenPass::after_projgen()
        {
            hook_trace.push_back("after_projgen");
            return true;
        }

        LanguageUnit_p BaseCodegenPass::codegen_device_type()
        {
            auto lu = std::make_shared<LanguageUnit>("device_type");
            *lu << "// 0: CUDA_GPU; 1: ROCM_GPU; 2: GENERIC_CPU; 3: HLSL; 4: GraphCore; 5: UNKNOWN\n";
            *lu << "extern \"C\" int get_device_type()\n{\n    return " << (int)device_type() << ";\n}\n";
            return lu;
        }

        LanguageUnit_p BaseCodegenPass::codegen_workspace_size(size_t total_bytes)
        {
            auto lu = std::make_shared<LanguageUnit>("workspace_size");
            *lu << "extern \"C\" int64_t get_workspace_size()\n{\n    return " << total_bytes << ";\n}\n";
            return lu;
        }

        // ---- HipCodegenPass ------------------------------------------------------------------------
        namespace
        {
            const char* RT_CPP = "nnfusion_rt.cpp";
            const char* RT_H = "nnfusion_rt.h";

            size_t align64(size_t n) { return (n + 63) & ~(size_t)63; }

            std::string ctype(const std::shared_ptr<descriptor::Tensor>& t)
            {
                return t->get_element_type().c_type_string();
            }
        } // namespace

        std::string HipCodegenPass::entry_signature(std::shared_ptr<TranslationUnit> tu, bool with_types) const
        {
            std::vector<std::string> params;
            for (auto& t : tu->arg)
                params.push_back((with_types ? ctype(t) + "* " : "") + t->get_name());
            for (auto& t : tu->out)
                params.push_back((with_types ? ctype(t) + "* " : "") + t->get_name());
            return join(params, ", ");
        }

        void HipCodegenPass::initialize(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu)
        {
            BaseCodegenPass::initialize(ctx, tu);
            m_tu = tu;
            m_pool = Pool();
            m_def_names.clear();
            m_globals = std::make_shared<LanguageUnit>("globals");
            m_defs = std::make_shared<LanguageUnit>("kernel_definitions");
            m_init = std::make_shared<LanguageUnit>("rocm_init_body");
            m_free = std::make_shared<LanguageUnit>("rocm_free_body");
            m_entry = std::make_shared<LanguageUnit>("kernel_entry_body");
            m_globals->require(kernels::header::hip);
            m_globals->require(kernels::header::stdio);
            m_globals->require(kernels::header::stdexcept);
            m_globals->require(kernels::header::sstream);
            m_globals->require(kernels::header::fstream);
            m_globals->require(kernels::header::nnf_hip_kernels);
            m_globals->require(kernels::macro::HIP_SAFE_CALL);
            m_globals->require(kernels::macro::NNF_HIP_CHECK);
            m_globals->require(kernels::declaration::typedef_int);
            m_globals->require(kernels::declaration::typedef_half);
            *m_globals << "#include \"" << RT_H << "\"\n";
            *m_globals << "static hipStream_t nnf_stream_0 = 0;\n";
            *m_globals << "static char* group_0_ROCM_GPU_0_memory_pool = nullptr;\n";
        }

        bool HipCodegenPass::collect_mem(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu)
        {
            BaseCodegenPass::collect_mem(ctx, tu);
            // Tensors that alias a kernel_entry argument: a Result forwards the caller's buffer to the
            // tensor it consumes (extern result memory), so the producing kernel writes straight into it.
            std::unordered_map<std::string, std::string> alias;
            for (auto& node : tu->m_graph->get_outputs())
            {
                auto src = node->get_input_tensor_ptr(0);
                if (!src->is_parameter() && !src->is_constant())
                    alias[src->get_name()] = node->get_output_tensor_ptr(0)->get_name();
            }
            m_init->indent = 1;
            m_free->indent = 1;
            m_entry->indent = 1;
            *m_init << "HIP_SAFE_CALL(hipSetDevice(0));\n";

            std::vector<std::pair<std::shared_ptr<descriptor::Tensor>, size_t>> pooled;
            auto place = [&](std::shared_ptr<descriptor::Tensor> t) {
                size_t off = m_pool.bytes;
                t->set_pool("group_0_ROCM_GPU_0_memory_pool");
                t->set_pool_offset(off);
                m_pool.bytes += align64(t->size());
                pooled.emplace_back(t, off);
            };
            for (auto& bb : tu->program)
                for (auto& ins : *bb)
                {
                    auto node = ins->getGNode();
                    if (node->is_parameter() || node->is_output())
                        continue;
                    if (node->is_constant())
                    {
                        auto t = node->get_output_tensor_ptr(0);
                        auto cop = std::dynamic_pointer_cast<op::Constant>(node->get_op_ptr());
                        NNFUSION_CHECK_NOT_NULLPTR(cop);
                        const std::string file = "Constant/" + t->get_name() + ".bin";
                        projgen->add_binary(file, cop->get_data_ptr(), cop->get_data_size());
                        *m_globals << "static " << ctype(t) << "* " << t->get_name() << " = nullptr;\n";
                        *m_init << "nnf_load_constant((void**)&" << t->get_name() << ", \"./" << file << "\", "
                                << t->size() << ");\n";
                        *m_free << "HIP_SAFE_CALL(hipFree(" << t->get_name() << "));\n";
                        continue;
                    }
                    for (size_t i = 0; i < node->get_output_size(); ++i)
                    {
                        auto t = node->get_output_tensor_ptr(i);
                        if (!alias.count(t->get_name()))
                            place(t);
                    }
                    if (auto k = ins->getKernel())
                        for (auto& t : k->m_context->tensors)
                            place(t);
                }
            if (m_pool.bytes > 0)
            {
                *m_init << "HIP_SAFE_CALL(hipMalloc((void**)&group_0_ROCM_GPU_0_memory_pool, " << m_pool.bytes << "));\n";
                *m_free << "HIP_SAFE_CALL(hipFree(group_0_ROCM_GPU_0_memory_pool));\n";
            }
            for (auto& pt : pooled)
            {
                *m_globals << "static " << ctype(pt.first) << "* " << pt.first->get_name() << " = nullptr;\n";
                *m_init << pt.first->get_name() << " = (" << ctype(pt.first) << "*)(group_0_ROCM_GPU_0_memory_pool + "
                        << pt.second << ");\n";
                // a tensor its kernel wants cleared (descriptor::Tensor::set_memset): nothing else lives at its place in
                // the pool, and the kernels that ask for this leave it cleared, so once, here, is enough (the reference
                // clears its memset pool at the top of every kernel_entry: cuda_codegen_pass.cpp:154-161)
                if (pt.first->is_memset())
                    *m_init << "HIP_SAFE_CALL(hipMemset(" << pt.first->get_name() << ", " << pt.first->get_memset_value() << ", "
                            << pt.first->size() << "));\n";
            }
            for (auto& kv : alias)
            {
                // the type of the aliased tensor equals the type of the Result tensor
                std::string type = "void";
                for (auto& node : tu->m_graph->get_outputs())
                    if (node->get_output_tensor_ptr(0)->get_name() == kv.second)
                        type = ctype(node->get_output_tensor_ptr(0));
                *m_entry << type << "* " << kv.first << " = " << kv.second << ";\n";
            }
            return true;
        }

        bool HipCodegenPass::collect_stream(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu)
        {
            BaseCodegenPass::collect_stream(ctx, tu);
            // one stream (the default of the reference unless -fnum_stream is given)
            for (auto& node : tu->m_graph->get_nodes())
                (*node)["Async_info_stream"] = std::string("nnf_stream_0");
            return true;
        }

        bool HipCodegenPass::collect_funcs(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu)
        {
            BaseCodegenPass::collect_funcs(ctx, tu);
            for (auto& bb : tu->program)
                for (auto& ins : *bb)
                {
                    auto node = ins->getGNode();
                    if (node->is_parameter() || node->is_constant())
                        continue;
                    if (node->is_output())
                    {
                        // a Result fed directly by a Parameter or Constant: copy (otherwise it is an alias)
                        auto src = node->get_input_tensor_ptr(0);
                        if (src->is_parameter() || src->is_constant())
                            *m_entry << "HIP_SAFE_CALL(hipMemcpyAsync(" << node->get_output_tensor_ptr(0)->get_name() << ", "
                                     << src->get_name() << ", " << src->size()
                                     << ", hipMemcpyDeviceToDevice, nnf_stream_0));\n";
                        continue;
                    }
                    auto kernel = ins->getKernel();
                    NNFUSION_CHECK_NOT_NULLPTR(kernel) << "no kernel selected for node " << node->get_name() << " ("
                                                       << node->get_op_type() << ")";
                    auto fu = kernel->get_or_emit_source(true);
                    NNFUSION_CHECK_NOT_NULLPTR(fu);
                    // identical signature + body => one definition shared by all its call sites
                    const std::string key = fu->signature_unit->get_code() + fu->body_unit->get_code();
                    std::string fname;
                    auto it = m_def_names.find(key);
                    if (it != m_def_names.end() && !kernel->is_static_function())
                    {
                        fname = it->second;
                    }
                    else
                    {
                        fname = fu->name_unit->get_code();
                        m_def_names[key] = fname;
                        *m_defs << fu->comment_unit->get_code();
                        *m_defs << fu->get_specialized_signature(fname) << "\n";
                        m_defs->block_begin();
                        *m_defs << fu->body_unit->get_code();
                        m_defs->block_end();
                        *m_defs << "\n";
                        m_defs->require(fu->dep_unit);
                        for (auto& kv : fu->dep_unit->local_symbol)
                            m_defs->require(kv.second);
                    }
                    *m_entry << fu->get_specialized_function_call(fname);
                }
            return true;
        }

        bool HipCodegenPass::modify_codegen()
        {
            BaseCodegenPass::modify_codegen();
            auto tu = m_tu;
            NNFUSION_CHECK_NOT_NULLPTR(tu);
            create_header_file(tu);

            auto helper = std::make_shared<LanguageUnit>("nnf_load_constant");
            auto& h = *helper;
            h << "\n// loads ./Constant/<tensor>.bin into device memory\n";
            h << "static void nnf_load_constant(void** dst, const char* path, size_t bytes)\n{\n";
            h << "    std::ifstream bin_file(path, std::ios::in | std::ios::binary);\n";
            h << "    if (bin_file.fail())\n    {\n        std::stringstream ss;\n        ss << \"Load \" << path << \" failed.\";\n"
                 "        throw std::runtime_error(ss.str());\n    }\n";
            h << "    char* tmp_mem = new char[bytes];\n    bin_file.read(tmp_mem, (std::streamsize)bytes);\n";
            h << "    HIP_SAFE_CALL(hipMalloc(dst, bytes));\n";
            h << "    HIP_SAFE_CALL(hipMemcpy(*dst, tmp_mem, bytes, hipMemcpyHostToDevice));\n";
            h << "    delete[] tmp_mem;\n}\n\n";

            auto rt = std::make_shared<LanguageUnit>("nnfusion_rt_functions");
            auto& r = *rt;
            r << "extern \"C\" void rocm_init()\n{\n" << m_init->get_code() << "}\n\n";
            r << "extern \"C\" void rocm_free()\n{\n" << m_free->get_code() << "}\n\n";
            r << "// the reference's ROCm code generator emits the cuda_ names; both are exported\n";
            r << "extern \"C\" void cuda_init()\n{\n    rocm_init();\n}\n\nextern \"C\" void cuda_free()\n{\n    rocm_free();\n}\n\n";
            r << "extern \"C\" int kernel_entry(" << entry_signature(tu, true) << ")\n{\n" << m_entry->get_code()
              << "    return 0;\n}\n\n";
            r << codegen_device_type()->get_code() << "\n" << codegen_workspace_size(m_pool.bytes)->get_code();

            projgen->add(RT_CPP, m_globals);
            projgen->add(RT_CPP, helper);
            projgen->add(RT_CPP, m_defs);
            projgen->add(RT_CPP, rt);
            create_main_file(tu);
            create_build_files();

            // para_info.json: what an external caller reads to drive kernel_entry
            // (written by ExtractGraphSignature in the reference, engine/pass/extract_graph_signature.cpp:160-236)
            auto pj = std::make_shared<LanguageUnit>("para_info");
            auto describe = [&](const std::vector<std::shared_ptr<descriptor::Tensor>>& ts, size_t base) {
                std::string text;
                for (size_t i = 0; i < ts.size(); ++i)
                {
                    std::ostringstream one;
                    one << "        \"" << ts[i]->get_name() << "\": {\"name\": \"" << ts[i]->get_name() << "\", \"id\": \"(("
                        << ctype(ts[i]) << "*)(args[" << (base + i) << "]))\", \"dtype\": \"" << ctype(ts[i])
                        << "\", \"shape\": [" << join(ts[i]->get_shape()) << "]}";
                    text += one.str() + (i + 1 < ts.size() ? ",\n" : "\n");
                }
                return text;
            };
            *pj << "{\n    \"input\": {\n" << describe(tu->arg, 0) << "    },\n    \"output\": {\n"
                << describe(tu->out, tu->arg.size()) << "    }\n}\n";
            projgen->add("para_info.json", pj);
            return true;
        }

        void HipCodegenPass::create_header_file(std::shared_ptr<TranslationUnit> tu)
        {
            auto lu = std::make_shared<LanguageUnit>("nnfusion_rt_header");
            *lu << "// Generated runtime interface.\n#pragma once\n#include <stdint.h>\n";
            *lu << "#ifndef NNF_HALF_DEFINED\n#define NNF_HALF_DEFINED\ntypedef _Float16 half;\n#endif\n";
            *lu << "extern \"C\" int kernel_entry(" << entry_signature(tu, true) << ");\n";
            *lu << "extern \"C\" void rocm_init();\nextern \"C\" void rocm_free();\n";
            *lu << "extern \"C\" void cuda_init();\nextern \"C\" void cuda_free();\n";
            *lu << "extern \"C\" int get_device_type();\nextern \"C\" int64_t get_workspace_size();\n";
            projgen->add(RT_H, lu);
        }

        void HipCodegenPass::create_main_file(std::shared_ptr<TranslationUnit> tu)
        {
            auto lu = std::make_shared<LanguageUnit>("main_test");
            auto& m = *lu;
            m << "// Stand-alone driver of the generated runtime: fills the inputs with ones, runs " << warmup_step
              << " warm-up and " << run_step << " timed calls of kernel_entry.\n";
            m << "#include <hip/hip_runtime.h>\n#include <stdio.h>\n#include <stdlib.h>\n#include <vector>\n#include <algorithm>\n";
            m << "#include \"nnfusion_rt.h\"\n\n";
            m << "#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf(\"%s failed: %s\\n\", #x, "
                 "hipGetErrorString(e)); return 1; } } while (0)\n\n";
            m << "int main(void)\n";
            m.block_begin();
            m << "rocm_init();\n";
            for (auto& t : tu->arg)
            {
                m << "// input argument\n";
                m << ctype(t) << "* " << t->get_name() << ";\n";
                m << "CHECK(hipMalloc((void**)&" << t->get_name() << ", " << t->size() << "));\n";
                m << "{\n    std::vector<" << ctype(t) << "> host(" << t->size(false) << ");\n";
                m << "    for (size_t i = 0; i < host.size(); ++i) host[i] = (" << ctype(t) << ")1;\n";
                m << "    CHECK(hipMemcpy(" << t->get_name() << ", host.data(), " << t->size() << ", hipMemcpyHostToDevice));\n}\n";
            }
            for (auto& t : tu->out)
            {
                m << "// output argument\n";
                m << ctype(t) << "* " << t->get_name() << ";\n";
                m << "CHECK(hipMalloc((void**)&" << t->get_name() << ", " << t->size() << "));\n";
            }
            m << "// warm up\n";
            m << "for (int i = 0; i < " << warmup_step << "; ++i)\n    kernel_entry(" << entry_signature(tu, false) << ");\n";
            m << "CHECK(hipDeviceSynchronize());\n";
            m << "hipEvent_t start, stop;\nCHECK(hipEventCreate(&start));\nCHECK(hipEventCreate(&stop));\n";
            m << "float ms_max = 0, ms_min = 1e30f, ms_total = 0;\n";
            m << "for (int i = 0; i < " << run_step << "; ++i)\n";
            m.block_begin();
            m << "CHECK(hipEventRecord(start, 0));\n";
            m << "kernel_entry(" << entry_signature(tu, false) << ");\n";
            m << "CHECK(hipEventRecord(stop, 0));\nCHECK(hipEventSynchronize(stop));\n";
            m << "float ms;\nCHECK(hipEventElapsedTime(&ms, start, stop));\n";
            m << "ms_max = std::max(ms, ms_max);\nms_min = std::min(ms, ms_min);\nms_total += ms;\n";
            m.block_end();
            for (auto& t : tu->out)
            {
                m << "{\n    std::vector<" << ctype(t) << "> host(" << t->size(false) << ");\n";
                m << "    CHECK(hipMemcpy(host.data(), " << t->get_name() << ", " << t->size() << ", hipMemcpyDeviceToHost));\n";
                m << "    printf(\"%s \\n\", \"" << t->get_name() << ":\");\n";
                m << "    for (size_t i = 0; i < std::min((size_t)10, host.size()); ++i) printf(\"%e \", (float)host[i]);\n";
                m << "    printf(\" .. (size = " << t->size(false) << ", ends with %e);\\n\", (float)host.back());\n}\n";
            }
            m << "printf(\"Summary: [min, max, mean] = [%f, %f, %f] ms\\n\", ms_min, ms_max, ms_total / " << run_step << ");\n";
            for (auto& t : tu->arg)
                m << "CHECK(hipFree(" << t->get_name() << "));\n";
            for (auto& t : tu->out)
                m << "CHECK(hipFree(" << t->get_name() << "));\n";
            m << "rocm_free();\nreturn 0;\n";
            m.block_end();
            projgen->add("main_test.cpp", lu);
        }

        void HipCodegenPass::create_build_files()
        {
            const std::string inc = kernels_include_dir.empty() ? "." : kernels_include_dir;
            const std::string lib = kernels_lib_dir.empty() ? "." : kernels_lib_dir;
            auto mk = std::make_shared<LanguageUnit>("makefile");
            *mk << "# Generated. HIP host code only: compiled by hipcc for gfx950, linked against the launcher library.\n";
            *mk << "HIPCC ?= /opt/rocm/bin/hipcc\n";
            *mk << "NNF_INC ?= " << inc << "\nNNF_LIB ?= " << lib << "\n";
            *mk << "FLAGS := -O2 -std=c++17 --offload-arch=gfx950 -I$(NNF_INC)\n\n";
            *mk << "all: libnnfusion_rocm_rt.so main_test\n\n";
            *mk << "libnnfusion_rocm_rt.so: nnfusion_rt.cpp nnfusion_rt.h\n";
            *mk << "\t$(HIPCC) $(FLAGS) -fPIC -shared -o $@ nnfusion_rt.cpp -L$(NNF_LIB) -lnnf_hip_kernels -Wl,-rpath,$(NNF_LIB)\n\n";
            *mk << "main_test: main_test.cpp libnnfusion_rocm_rt.so\n";
            *mk << "\t$(HIPCC) $(FLAGS) -o $@ main_test.cpp -L. -lnnfusion_rocm_rt -Wl,-rpath,'$$ORIGIN' -L$(NNF_LIB) "
                   "-lnnf_hip_kernels -Wl,-rpath,$(NNF_LIB)\n\n";
            *mk << "clean:\n\trm -f libnnfusion_rocm_rt.so main_test\n";
            projgen->add("Makefile", mk);

            auto cm = std::make_shared<LanguageUnit>("cmakelists");
            *cm << "project(main_test)\ncmake_minimum_required(VERSION 3.5)\n";
            *cm << "set(CMAKE_CXX_COMPILER /opt/rocm/bin/hipcc)\n";
            *cm << "set(CMAKE_CXX_FLAGS \"${CMAKE_CXX_FLAGS} -O2 -std=c++17 --offload-arch=gfx950\")\n";
            *cm << "include_directories(" << inc << ")\nlink_directories(" << lib << ")\n";
            *cm << "add_library(nnfusion_rocm_rt SHARED nnfusion_rt.cpp)\ntarget_link_libraries(nnfusion_rocm_rt nnf_hip_kernels)\n";
            *cm << "add_executable(main_test main_test.cpp)\ntarget_link_libraries(main_test nnfusion_rocm_rt nnf_hip_kernels)\n";
            projgen->add("CMakeLists.txt", cm);
        }

        bool HipCodegenPass::after_projgen()
        {
            BaseCodegenPass::after_projgen();
            return true; // nothing to post-process: the text written is already HIP
        }

    } // namespace codegen

    bool ROCmEngine::run_on_graph(std::shared_ptr<graph::Graph> graph)
    {
        if (quant_epilogue_fusion)
        {
            pass::graph::QuantEpilogueFusionPass fusion;
            NNFUSION_CHECK(fusion.run_on_graph(graph));
        }
        if (quant_gemm_fusion)
        {
            pass::graph::QuantGemmFusionPass merge;
            NNFUSION_CHECK(merge.run_on_graph(graph));
        }
        pass::graph::DefaultGNodeDeviceDispatcher dispatcher(ROCM_GPU);
        NNFUSION_CHECK(dispatcher.run_on_graph(graph));
        if (kernel_selection)
        {
            profiler::HipDefaultRuntime runtime(pass.kernels_include_dir, pass.kernels_lib_dir);
            pass::graph::ProfilingBasedKernelSelector profiling;
            profiling.working_dir = kernel_profiling_dir;
            profiling.runtime_times = kernel_profiling_runs;
            profiling.prepare_only = kernel_selection_prepare_only;
            NNFUSION_CHECK(profiling.run_on_graph(graph, runtime));
            if (kernel_selection_prepare_only)
                return true;
        }
        pass::graph::DefaultKernelSelector selector;
        NNFUSION_CHECK(selector.run_on_graph(graph));
        // Only the quantized products (and Slice) have emitters for this device.  Element-wise operators of an imported
        // model must have been absorbed by the fusion passes above; one that was not (a gate product with a second
        // consumer, a bias added after the residual, a normalisation that feeds another operator ...) is named here,
        // before any code is written.
        {
            std::string unserved;
            for (auto& node : graph->get_ordered_ops())
            {
                if (node->is_parameter() || node->is_constant() || node->is_output())
                    continue;
                if (!(*node)["Kernel_Selection_Result"].is_valid())
                    unserved += (unserved.empty() ? "" : ", ") + node->get_name() + " (" + node->get_op_type() + ")";
            }
            NNFUSION_CHECK(unserved.empty())
                << "no " << get_device_str(ROCM_GPU) << " kernel for: " << unserved
                << "; the quantized fusion passes did not absorb these operators, and only QuantDot, QuantDotW8A8, "
                   "FusedQuantMLP and Slice have emitters";
        }
        auto tu = visit_graph(graph);
        auto ctx = std::make_shared<InterpreterContext>();
        ctx->m_graph = graph;
        return pass.run(ctx, tu);
    }
} // namespace nnfusion
