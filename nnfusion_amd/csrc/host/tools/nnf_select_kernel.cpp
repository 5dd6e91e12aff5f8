// nnf_select_kernel: profiling-based kernel selection for one QuantDot node, the way the reference's
// ProfilingBasedKernelSelector does it for its white-listed operators
// (src/nnfusion/engine/pass/graph/kernel_selection.cpp:21-137): every registered emitter that accepts the
// node goes through the single-kernel harness and the fastest wins.
//
//   nnf_select_kernel prepare <dir> M N K <include_dir> <lib_dir>   generate and compile the harnesses (no device)
//   nnf_select_kernel run     <dir> M N K <include_dir> <lib_dir>   run them (objects built by `prepare` are
//                                                                    reused), print one JSON line
#include "../nnf_datagen.h"
#include "nnfusion/core/operators/generic_op/generic_op.hpp"
#include "nnfusion/engine/pass/graph/kernel_selection.hpp"

#include <cmath>
#include <cstdlib>
#include <cstring>

using namespace nnfusion;

namespace
{
    float half_bits_to_float(uint16_t h)
    {
        const uint32_t sign = (uint32_t)(h & 0x8000) << 16;
        uint32_t exp = (h >> 10) & 0x1F, man = h & 0x3FF, bits;
        if (exp == 0)
        {
            if (man == 0)
                bits = sign;
            else
            {
                int e = -1;
                do
                {
                    ++e;
                    man <<= 1;
                } while (!(man & 0x400));
                bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FF) << 13);
            }
        }
        else if (exp == 31)
            bits = sign | 0x7F800000u | (man << 13);
        else
            bits = sign | ((exp + 112) << 23) | (man << 13);
        float f;
        memcpy(&f, &bits, 4);
        return f;
    }
} // namespace

int main(int argc, char** argv)
{
    if (argc < 8)
    {
        fprintf(stderr, "usage: %s <prepare|run> <dir> M N K <include_dir> <lib_dir> [runs]\n", argv[0]);
        return 2;
    }
    const std::string mode = argv[1], dir = argv[2];
    const size_t M = strtoul(argv[3], nullptr, 10), N = strtoul(argv[4], nullptr, 10), K = strtoul(argv[5], nullptr, 10);
    try
    {
        auto g = std::make_shared<graph::Graph>();
        auto a = g->add_node_and_edge(std::make_shared<op::Parameter>(element::f16, Shape{M, K}), graph::GNodeVector{});
        std::vector<uint8_t> wq(N * K / 2, 0x88);
        std::vector<uint16_t> sc(N * (K / 128), 0x2000);
        auto w = g->add_node_and_edge(std::make_shared<op::Constant>(element::u8, Shape{N, K / 2}, wq.data()), graph::GNodeVector{});
        auto s = g->add_node_and_edge(std::make_shared<op::Constant>(element::f16, Shape{N, K / 128}, sc.data()), graph::GNodeVector{});
        auto dot = g->add_node_and_edge(std::make_shared<op::GenericOp>("linear", "QuantDot", op::OpConfig::any()), {a, w, s});
        g->add_node_and_edge(std::make_shared<op::Result>(), {dot});
        pass::graph::DefaultGNodeDeviceDispatcher().run_on_graph(g);

        profiler::HipDefaultRuntime rt(argv[6], argv[7]);
        pass::graph::ProfilingBasedKernelSelector sel;
        sel.working_dir = dir;
        if (argc > 8)
            sel.runtime_times = strtoul(argv[8], nullptr, 10);
        if (mode == "prepare")
        {
            if (!rt.check_env())
            {
                fprintf(stderr, "hipcc not found\n");
                return 1;
            }
            size_t built = 0;
            for (auto& pc : sel.contexts(dot, ROCM_GPU, rt))
            {
                if (!rt.compile(pc))
                    return 1;
                ++built;
            }
            printf("{\"prepared\": %zu}\n", built);
            return 0;
        }
        std::vector<pass::graph::ProfilingBasedKernelSelector::Timing> timings;
        std::vector<std::vector<uint8_t>> outs;
        auto best = sel.profiling_best(dot, ROCM_GPU, rt, &timings, &outs);
        // how far the candidates' results are apart (they ran on the same inputs)
        double max_diff = 0.0, max_ref = 0.0;
        for (size_t c = 1; c < outs.size(); ++c)
            for (size_t i = 0; i + 1 < outs[c].size(); i += 2)
            {
                uint16_t x, y;
                memcpy(&x, &outs[0][i], 2);
                memcpy(&y, &outs[c][i], 2);
                const double fx = half_bits_to_float(x), fy = half_bits_to_float(y);
                max_diff = std::max(max_diff, std::fabs(fx - fy));
                max_ref = std::max(max_ref, std::fabs(fx));
            }
        printf("{\"M\": %zu, \"N\": %zu, \"K\": %zu, \"candidates\": [", M, N, K);
        for (size_t i = 0; i < timings.size(); ++i)
            printf("%s{\"kernel\": \"%s\", \"ms\": %.6f}", i ? ", " : "", timings[i].kernel_type.c_str(), timings[i].ms);
        printf("], \"best\": \"%s\", \"ran\": %zu, \"max_abs_diff\": %.6g, \"max_abs_ref\": %.6g}\n",
               best.second ? best.second->get_kernel_type().c_str() : "", outs.size(), max_diff, max_ref);
        return best.second ? 0 : 1;
    }
    catch (const std::exception& e)
    {
        fprintf(stderr, "nnf_select_kernel: %s\n", e.what());
        return 1;
    }
}
