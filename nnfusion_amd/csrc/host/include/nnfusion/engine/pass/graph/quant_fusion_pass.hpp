// Graph passes that produce the shapes the quantized kernels are built for.  Counterparts, for the
// quantized operators, of the reference's Dot-centred rewrites:
//   * GEMMFuseOptimizer (src/nnfusion/engine/pass/graph/gemm_fusion_pass.cpp:61-530): Dots that share an
//     input become one wide Dot followed by Slices ("fused QKV" 3 x 4096 -> 12288);
//   * the subgraph fusion optimizers (e.g. subgraph_fusion_optimizer/matmuladd_fusion_optimizer.cpp:8-93:
//     MatMul + Add -> MatMulAdd), here: RMSNorm -> QuantDot, QuantDot -> +bias / +residual,
//     SiLU(QuantDot_gate) * QuantDot_up -> one QuantDot with the gate and up weights stacked, and the whole
//     block x + down(SiLU(gate(n)) * up(n)), n = RMSNorm(x), -> FusedQuantMLP.
// The graph of this build is append-only, so a pass rebuilds the graph instead of editing it in place and
// swaps the caller's pointer; nodes that are no longer reachable from a Result are dropped.
#pragma once

#include "nnfusion/core/graph/gnode.hpp"

namespace nnfusion
{
    namespace pass
    {
        namespace graph
        {
            // src/nnfusion/engine/pass/graph/graph_pass_base.hpp:14-28
            class GraphPassBase
            {
            public:
                virtual ~GraphPassBase() = default;
                virtual bool run_on_graph(std::shared_ptr<nnfusion::graph::Graph>& graph) { return true; }
            };

            // Folds prologues / epilogues into QuantDot and whole MLP blocks into FusedQuantMLP.
            // Runs to a fixed point; `fused` counts the rewrites of the last run.
            class QuantEpilogueFusionPass : public GraphPassBase
            {
            public:
                bool run_on_graph(std::shared_ptr<nnfusion::graph::Graph>& graph) override;
                size_t fused = 0;
            };

            // Merges QuantDot nodes that read the same activations (same prologue, no epilogue, constant
            // weights) into one QuantDot over the row-concatenated weights, followed by one Slice per
            // original node.  Off by default in the engine, like -fgemm_fusion in the reference
            // (gemm_fusion_pass.cpp:15).
            class QuantGemmFusionPass : public GraphPassBase
            {
            public:
                bool run_on_graph(std::shared_ptr<nnfusion::graph::Graph>& graph) override;
                size_t merged_groups = 0;
            };
        } // namespace graph
    } // namespace pass
} // namespace nnfusion
