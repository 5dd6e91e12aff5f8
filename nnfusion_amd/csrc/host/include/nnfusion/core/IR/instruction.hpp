// ir::Instruction / Program / TranslationUnit: what the graph visitor hands to the codegen passes
// (src/nnfusion/core/IR/instruction.{hpp,cpp}, src/nnfusion/engine/device/reversed_dfs_visitor.cpp:233-265).
#pragma once

#include "nnfusion/core/kernels/kernel_emitter.hpp"

namespace nnfusion
{
    namespace ir
    {
        class Instruction
        {
        public:
            using Pointer = std::shared_ptr<Instruction>;
            // pulls the emitter out of the node's "Kernel_Selection_Result" tag
            void setGNode(std::shared_ptr<graph::GNode> gnode);
            std::shared_ptr<graph::GNode> getGNode() const { return m_gnode; }
            kernels::KernelEmitter::Pointer getKernel() const { return m_kernel; }
            void setKernel(kernels::KernelEmitter::Pointer k) { m_kernel = k; }

        private:
            std::shared_ptr<graph::GNode> m_gnode;
            kernels::KernelEmitter::Pointer m_kernel;
        };
        using BasicBlock = std::vector<Instruction::Pointer>;
        using Program = std::vector<std::shared_ptr<BasicBlock>>;
    } // namespace ir

    struct InterpreterContext
    {
        std::shared_ptr<graph::Graph> m_graph;
    };

    struct TranslationUnit
    {
        std::shared_ptr<graph::Graph> m_graph;
        ir::Program program;
        // graph inputs (Parameter outputs) and outputs (Result inputs), in kernel_entry order
        std::vector<std::shared_ptr<descriptor::Tensor>> arg, out;
    };

    // One basic block, one instruction per node, in topological order
    // (the product of ReversedDFSVisitor::run_on_graph).
    std::shared_ptr<TranslationUnit> visit_graph(std::shared_ptr<graph::Graph> graph);
} // namespace nnfusion
