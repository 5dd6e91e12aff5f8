// BaseCodegenPass: the template method every code generator follows
// (src/nnfusion/engine/pass/codegen/base_codegen_pass.hpp:17-105, .cpp:17-33):
//   initialize -> collect_mem -> collect_stream -> collect_funcs -> modify_codegen -> projgen->codegen()
//   -> after_projgen -> exit(0)
// and HipCodegenPass, the gfx950 generator: it writes HIP host code directly (no CUDA text, no
// hipify post-pass, no CUDA-compat header) in place of RocmCodegenPass (rocm_codegen_pass.cpp:24-295).
#pragma once

#include "nnfusion/core/IR/instruction.hpp"

namespace nnfusion
{
    namespace codegen
    {
        // The generated project as an ordered set of files; each file is a list of language units.
        // Units are written dependencies first: header:: < macro:: < declaration:: < everything else
        // (src/nnfusion/engine/pass/codegen/codegenerator.cpp:140-303).
        class CodeGenerator
        {
        public:
            using Pointer = std::shared_ptr<CodeGenerator>;
            CodeGenerator(const std::string& codegen_folder, const std::string& kernel_suffix)
                : m_codegen_folder(codegen_folder)
                , m_kernel_suffix(kernel_suffix)
            {
            }
            // append a unit to a file of the project (relative path); required units are pulled in
            void add(const std::string& file, LanguageUnit_p lu);
            void change_codegen_folder(const std::string& f) { m_codegen_folder = f; }
            void change_kernel_suffix(const std::string& s) { m_kernel_suffix = s; }
            const std::string& get_codegen_folder() const { return m_codegen_folder; }
            // binary side files (Constant/<name>.bin)
            void add_binary(const std::string& file, const void* data, size_t bytes);
            // write everything below the codegen folder; returns false on I/O failure
            bool codegen();
            // text a file would get (tests)
            std::string render(const std::string& file) const;
            std::vector<std::string> files() const;

        private:
            std::string m_codegen_folder, m_kernel_suffix;
            std::vector<std::string> m_order;
            std::map<std::string, std::vector<LanguageUnit_p>> m_files;
            std::map<std::string, std::vector<uint8_t>> m_binaries;
        };

        class BaseCodegenPass
        {
        public:
            BaseCodegenPass(const std::string& codegen_folder = "./nnfusion_rt/base_codegen/",
                            const std::string& kernel_folder = "./nnfusion_rt/base_codegen/",
                            const std::string kernel_suffix = ".cpp")
                : projgen(new CodeGenerator(codegen_folder, kernel_suffix))
                , m_codegen_folder(codegen_folder)
                , m_kernel_folder(kernel_folder)
                , m_kernel_suffix(kernel_suffix)
            {
            }
            virtual ~BaseCodegenPass() = default;
            virtual bool run(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu);
            // The reference ends the process after code generation; tests and embedding callers switch it off.
            bool exit_after_codegen = true;
            // order in which the hooks ran (observable by tests)
            std::vector<std::string> hook_trace;
            CodeGenerator::Pointer projgen;

        protected:
            virtual void initialize(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu);
            virtual bool collect_funcs(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu);
            virtual bool collect_mem(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu);
            virtual bool collect_stream(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu);
            virtual bool modify_codegen();
            virtual bool after_projgen();
            virtual NNFusion_DeviceType device_type() { return UNKNOWN; }
            // "int get_device_type()" / "int64_t get_workspace_size()" of the generated runtime
            LanguageUnit_p codegen_device_type();
            LanguageUnit_p codegen_workspace_size(size_t total_bytes);
            virtual void change_codegen_folder(const std::string& f)
            {
                m_codegen_folder = f;
                projgen->change_codegen_folder(f);
            }
            const std::string& get_codegen_folder() const { return m_codegen_folder; }

            std::string m_codegen_folder, m_kernel_folder, m_kernel_suffix;
        };

        class HipCodegenPass : public BaseCodegenPass
        {
        public:
            explicit HipCodegenPass(const std::string& codegen_folder = "./nnfusion_rt/rocm_codegen/")
                : BaseCodegenPass(codegen_folder, codegen_folder, ".cpp")
            {
            }
            // warm-up and timed iterations of the generated main_test (the reference's -fwarmup_step / -frun_step)
            int warmup_step = 5, run_step = 100;
            // where the generated Makefile / CMakeLists.txt find nnf_hip_kernels.h and libnnf_hip_kernels.so
            std::string kernels_include_dir, kernels_lib_dir;

        protected:
            NNFusion_DeviceType device_type() override { return ROCM_GPU; }
            void initialize(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu) override;
            bool collect_mem(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu) override;
            bool collect_stream(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu) override;
            bool collect_funcs(std::shared_ptr<InterpreterContext> ctx, std::shared_ptr<TranslationUnit> tu) override;
            bool modify_codegen() override;
            bool after_projgen() override;

        private:
            void create_header_file(std::shared_ptr<TranslationUnit> tu);
            void create_main_file(std::shared_ptr<TranslationUnit> tu);
            void create_build_files();
            std::string entry_signature(std::shared_ptr<TranslationUnit> tu, bool with_types) const;

            struct Pool
            {
                size_t bytes = 0;
            };
            Pool m_pool;                          // intermediate tensors: one 64-byte aligned bump pool
            LanguageUnit_p m_init, m_free, m_entry; // bodies of rocm_init(), rocm_free(), kernel_entry()
            LanguageUnit_p m_defs;                // kernel definitions, de-duplicated by signature + body
            LanguageUnit_p m_globals;             // global pointers of constants / intermediates
            std::map<std::string, std::string> m_def_names; // "signature+body" -> function name
            std::shared_ptr<TranslationUnit> m_tu;
        };
    } // namespace codegen

    // The ROCm engine reduced to the passes this path needs (src/nnfusion/engine/device/rocm.cpp:41-90):
    // quantized-op fusion passes -> device dispatch -> kernel selection -> visitor -> HipCodegenPass.
    class ROCmEngine
    {
    public:
        explicit ROCmEngine(const std::string& codegen_folder = "./nnfusion_rt/rocm_codegen/")
            : pass(codegen_folder)
        {
        }
        bool run_on_graph(std::shared_ptr<graph::Graph> graph);
        codegen::HipCodegenPass pass;
        bool quant_epilogue_fusion = true; // QuantEpilogueFusionPass
        bool quant_gemm_fusion = false;    // QuantGemmFusionPass (off by default, like -fgemm_fusion)
        // ProfilingBasedKernelSelector ahead of the default selector (off by default, like -fkernel_selection):
        // needs hipcc and a GPU at compile time; harness objects already in kernel_profiling_dir are reused
        bool kernel_selection = false;
        std::string kernel_profiling_dir = "./kernel_profiling/";
        size_t kernel_profiling_runs = 100;
        bool kernel_selection_prepare_only = false; // build the harnesses and stop before code generation
    };
} // namespace nnfusion
