// Single-kernel harness: source generation, hipcc compile, dlopen and run of
//   extern "C" double <name>_entry(void** args, void** outputs)
// for one emitted kernel (the protocol of the reference's profiler runtimes; the ROCm one there
// generates CUDA text, rewrites it with hipify and compiles with hipcc, rocm_runtime.cpp:20-106 --
// here the emitted text is HIP host code from the start).
#include "nnfusion/engine/profiler/hip_runtime.hpp"

#include <cstdio>
#include <cstdlib>
#include <dlfcn.h>
#include <fstream>
#include <iterator>
#include <sys/stat.h>
#include <unistd.h>

namespace nnfusion
{
    namespace profiler
    {
        bool HipDefaultRuntime::check_env() const { return access("/opt/rocm/bin/hipcc", X_OK) == 0; }

        bool HipDefaultRuntime::codegen(ProfilingContext::Pointer ke)
        {
            auto kernel = ke->kernel;
            auto fu = kernel->get_or_emit_source();
            if (!fu)
                return false;
            auto& ctx = kernel->m_context;
            const std::string name = fu->name_unit->get_code();
            ke->entry_name = name + "_entry";

            LanguageUnit src("profiler_source");
            src << fu->dep_unit->collect_required_code();
            src << "#include <vector>\n\n";
            src << "#define PROF_CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { fprintf(stderr, \"%s: %s\\n\", #x, "
                   "hipGetErrorString(e)); return -1.0; } } while (0)\n\n";
            src << fu->comment_unit->get_code();
            src << "static " << fu->get_specialized_signature() << "\n";
            src.block_begin();
            src << fu->body_unit->get_code();
            src.block_end();
            src << "\n";

            struct Buf
            {
                std::string type, host, dev;
                size_t bytes;
                int dir; // 0 input, 1 output, 2 scratch
            };
            std::vector<Buf> bufs;
            for (size_t i = 0; i < ctx->inputs.size(); ++i)
                bufs.push_back({ctx->inputs[i]->get_element_type().c_type_string(), "input" + std::to_string(i) + "_host",
                                "input" + std::to_string(i), ctx->inputs[i]->size(), 0});
            for (size_t i = 0; i < ctx->outputs.size(); ++i)
                bufs.push_back({ctx->outputs[i]->get_element_type().c_type_string(),
                                "output" + std::to_string(i) + "_host", "output" + std::to_string(i),
                                ctx->outputs[i]->size(), 1});
            for (auto& t : ctx->tensors) // dir 3: scratch that its kernel wants cleared
                bufs.push_back({t->get_element_type().c_type_string(), "", t->get_name(), t->size(), t->is_memset() ? 3 : 2});

            std::vector<std::string> host_params, call_args{"stream"};
            for (auto& b : bufs)
            {
                if (b.dir < 2)
                    host_params.push_back(b.type + "* " + b.host);
                call_args.push_back(b.dev);
            }
            src << "extern \"C\" double " << name << "_host(" << join(host_params, ", ") << ")\n";
            src.block_begin();
            src << "hipStream_t stream = 0;\n";
            for (auto& b : bufs)
            {
                src << b.type << "* " << b.dev << " = nullptr;\n";
                src << "PROF_CHECK(hipMalloc((void**)&" << b.dev << ", " << std::max<size_t>(b.bytes, 16) << "));\n";
                if (b.dir == 0 && b.bytes)
                    src << "PROF_CHECK(hipMemcpy(" << b.dev << ", " << b.host << ", " << b.bytes << ", hipMemcpyHostToDevice));\n";
                if (b.dir == 3)
                    src << "PROF_CHECK(hipMemset(" << b.dev << ", 0, " << std::max<size_t>(b.bytes, 16) << "));\n";
            }
            const std::string call = name + "(" + join(call_args, ", ") + ");\n";
            src << "try\n";
            src.block_begin();
            src << "for (size_t i = 0; i < " << ke->warmup_times << "; ++i)\n    " << call;
            src.block_end();
            src << "catch (const std::exception& e)\n";
            src.block_begin();
            src << "fprintf(stderr, \"%s\\n\", e.what());\nreturn -1.0;\n";
            src.block_end();
            src << "hipEvent_t start, stop;\nPROF_CHECK(hipEventCreate(&start));\nPROF_CHECK(hipEventCreate(&stop));\n";
            src << "PROF_CHECK(hipEventRecord(start, stream));\n";
            src << "for (size_t i = 0; i < " << ke->runtime_times << "; ++i)\n    " << call;
            src << "PROF_CHECK(hipEventRecord(stop, stream));\nPROF_CHECK(hipEventSynchronize(stop));\n";
            src << "float ms = 0;\nPROF_CHECK(hipEventElapsedTime(&ms, start, stop));\n";
            for (auto& b : bufs)
                if (b.dir == 1 && b.bytes)
                    src << "PROF_CHECK(hipMemcpy(" << b.host << ", " << b.dev << ", " << b.bytes << ", hipMemcpyDeviceToHost));\n";
            for (auto& b : bufs)
                src << "PROF_CHECK(hipFree(" << b.dev << "));\n";
            src << "return (double)ms / " << std::max<size_t>(ke->runtime_times, 1) << ";\n";
            src.block_end();
            src << "\n";

            src << "extern \"C\" double " << ke->entry_name << "(void** args, void** outputs)\n";
            src.block_begin();
            std::vector<std::string> fwd;
            size_t in_i = 0, out_i = 0;
            for (auto& b : bufs)
            {
                if (b.dir == 0)
                    fwd.push_back("(" + b.type + "*)args[" + std::to_string(in_i++) + "]");
                else if (b.dir == 1)
                    fwd.push_back("(" + b.type + "*)outputs[" + std::to_string(out_i++) + "]");
            }
            src << "return " << name << "_host(" << join(fwd, ", ") << ");\n";
            src.block_end();
            ke->source_code = src.get_code();
            return true;
        }

        bool HipDefaultRuntime::compile(ProfilingContext::Pointer ke)
        {
            if (ke->source_code.empty() && !codegen(ke))
                return false;
            std::string dir = ke->working_dir;
            if (dir.empty())
                dir = "./";
            if (dir.back() != '/')
                dir += '/';
            mkdir(dir.c_str(), 0755);
            ke->source_path = dir + ke->entry_name + ".cpp";
            ke->object_path = dir + "lib" + ke->entry_name + ".so";
            {
                // an object built earlier from the same source (e.g. ahead of time, on a host without the
                // device) is kept
                std::ifstream old_src(ke->source_path);
                if (old_src.is_open())
                {
                    std::string old_text((std::istreambuf_iterator<char>(old_src)), std::istreambuf_iterator<char>());
                    if (old_text == ke->source_code && access(ke->object_path.c_str(), R_OK) == 0)
                        return true;
                }
            }
            {
                std::ofstream f(ke->source_path, std::ios::trunc);
                if (!f.good())
                    return false;
                f << ke->source_code;
            }
            std::string cmd = "/opt/rocm/bin/hipcc -O2 -std=c++17 --offload-arch=gfx950 -fPIC -shared -I" + m_include_dir +
                              " -o " + ke->object_path + " " + ke->source_path + " -L" + m_lib_dir +
                              " -lnnf_hip_kernels -Wl,-rpath," + m_lib_dir + " 2>&1";
            FILE* p = popen(cmd.c_str(), "r");
            if (!p)
                return false;
            std::string out;
            char buf[512];
            while (fgets(buf, sizeof(buf), p))
                out += buf;
            int rc = pclose(p);
            if (rc != 0)
            {
                NNFUSION_LOG(ERROR) << "hipcc failed for " << ke->source_path << ":\n" << out;
                return false;
            }
            return true;
        }

        double HipDefaultRuntime::execute(ProfilingContext::Pointer ke, void** inputs, void** outputs)
        {
            if (!ke->entry_point)
            {
                if (ke->object_path.empty() && !compile(ke))
                    return -1.0;
                ke->handle = dlopen(ke->object_path.c_str(), RTLD_NOW | RTLD_LOCAL);
                if (!ke->handle)
                {
                    NNFUSION_LOG(ERROR) << "dlopen failed: " << dlerror();
                    return -1.0;
                }
                ke->entry_point = reinterpret_cast<double (*)(void**, void**)>(dlsym(ke->handle, ke->entry_name.c_str()));
                if (!ke->entry_point)
                    return -1.0;
            }
            return ke->entry_point(inputs, outputs);
        }
    } // namespace profiler
} // namespace nnfusion
