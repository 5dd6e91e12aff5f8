// QuantEpilogueFusionPass / QuantGemmFusionPass and the few element-wise operators they match on.
// See include/nnfusion/engine/pass/graph/quant_fusion_pass.hpp for what they stand for in the reference.
#include "nnfusion/engine/pass/graph/quant_fusion_pass.hpp"

#include "nnfusion/core/operators/generic_op/generic_op.hpp"

#include <cstring>
#include <functional>
#include <map>
#include <set>
#include <sstream>

using namespace nnfusion;
using nnfusion::graph::GNode;
using nnfusion::graph::GNodeVector;
using nnfusion::graph::Graph;

// ---- operators the patterns are written in -------------------------------------------------------------
// RMSNorm has no operator in the reference (its LayerNorm is cuda_gpu/cuda_langunit.cpp:618); Add / Multiply /
// Sigmoid are the element-wise ops of cuda_gpu/cuda_kernelops.hpp:408,416,447-451; Swish is x * sigmoid(x) as
// one node; Slice keeps a range of the last axis (the reference's op::Slice with unit strides).
REGISTER_OP(RMSNorm).attr<double>("eps", 1e-6).infershape([](std::shared_ptr<GNode> gnode) -> void {
    auto gop = std::dynamic_pointer_cast<op::GenericOp>(gnode->get_op_ptr());
    OP_VALIDATION(gop, gnode->get_input_size() == 2) << "inputs: x, gamma";
    OP_VALIDATION(gop, shape_size(gnode->get_input_shape(1)) == gnode->get_input_shape(0).back()) << "gamma is [K]";
    gnode->set_output_type_and_shape(0, gnode->get_input_element_type(0), gnode->get_input_shape(0));
});

namespace
{
    void infer_binary(std::shared_ptr<GNode> gnode)
    {
        auto gop = std::dynamic_pointer_cast<op::GenericOp>(gnode->get_op_ptr());
        OP_VALIDATION(gop, gnode->get_input_size() == 2) << "two inputs";
        const Shape& a = gnode->get_input_shape(0);
        const Shape& b = gnode->get_input_shape(1);
        // same shape, or the second operand is a row broadcast over the leading axes
        OP_VALIDATION(gop, a == b || (b.size() == 1 && b[0] == a.back()) || (a.size() == 1 && a[0] == b.back()))
            << "shapes do not broadcast";
        gnode->set_output_type_and_shape(0, gnode->get_input_element_type(0), a.size() >= b.size() ? a : b);
    }
    void infer_unary(std::shared_ptr<GNode> gnode)
    {
        auto gop = std::dynamic_pointer_cast<op::GenericOp>(gnode->get_op_ptr());
        OP_VALIDATION(gop, gnode->get_input_size() == 1) << "one input";
        gnode->set_output_type_and_shape(0, gnode->get_input_element_type(0), gnode->get_input_shape(0));
    }
} // namespace

REGISTER_OP(Add).infershape(infer_binary);
REGISTER_OP(Multiply).infershape(infer_binary);
REGISTER_OP(Sigmoid).infershape(infer_unary);
REGISTER_OP(Swish).infershape(infer_unary);
REGISTER_OP(Slice).attr<int>("begin", 0).attr<int>("end", 0).infershape([](std::shared_ptr<GNode> gnode) -> void {
    auto gop = std::dynamic_pointer_cast<op::GenericOp>(gnode->get_op_ptr());
    OP_VALIDATION(gop, gnode->get_input_size() == 1) << "one input";
    Shape s = gnode->get_input_shape(0);
    const int b = gop->localOpConfig.getRoot()["begin"].get<int>(), e = gop->localOpConfig.getRoot()["end"].get<int>();
    OP_VALIDATION(gop, !s.empty() && 0 <= b && b < e && (size_t)e <= s.back()) << "range outside the last axis";
    s.back() = (size_t)(e - b);
    gnode->set_output_type_and_shape(0, gnode->get_input_element_type(0), s);
});

namespace
{
    using NodeOut = std::pair<std::shared_ptr<GNode>, int>;

    std::shared_ptr<op::GenericOp> generic(const std::shared_ptr<GNode>& n)
    {
        return std::dynamic_pointer_cast<op::GenericOp>(n->get_op_ptr());
    }
    bool is_op(const std::shared_ptr<GNode>& n, const char* type) { return n->get_op_type() == type; }
    NodeOut input_of(const std::shared_ptr<GNode>& n, size_t i)
    {
        const auto& e = n->get_in_edge(i);
        return {e.src, e.src_output};
    }

    struct QuantDotInfo
    {
        bool rms = false, has_bias = false, has_res = false, gate = false, has_z = false;
        int group = 128, zp = 8, bits = 4;
        double eps = 1e-6;
        NodeOut a, wq, s, z, gamma, bias, res;
        bool same_block_parameters(const QuantDotInfo& o) const
        {
            return group == o.group && bits == o.bits && has_z == o.has_z && (has_z || zp == o.zp);
        }
    };
    bool quant_dot_info(const std::shared_ptr<GNode>& n, QuantDotInfo& q)
    {
        if (!is_op(n, "QuantDot"))
            return false;
        auto& cfg = generic(n)->localOpConfig.getRoot();
        q.rms = cfg["rms_norm"].get<bool>();
        q.has_bias = cfg["has_bias"].get<bool>();
        q.has_res = cfg["has_residual"].get<bool>();
        q.gate = cfg["act"].get<std::string>() == "silu_gate";
        q.group = cfg["group_size"].get<int>();
        q.zp = cfg["zero_point"].get<int>();
        q.bits = cfg["bits"].get<int>();
        q.eps = cfg["rms_eps"].get<double>();
        q.has_z = cfg["has_zero_points"].get<bool>();
        // (every block parameter has fused forms: the specialised kernels' own, or the nodes run one after the other
        // inside one call of the launcher library)
        size_t i = 0;
        q.a = input_of(n, i++);
        q.wq = input_of(n, i++);
        q.s = input_of(n, i++);
        if (q.has_z)
            q.z = input_of(n, i++);
        if (q.rms)
            q.gamma = input_of(n, i++);
        if (q.has_bias)
            q.bias = input_of(n, i++);
        if (q.has_res)
            q.res = input_of(n, i++);
        return true;
    }
    op::OpConfig::any quant_dot_config(const QuantDotInfo& q)
    {
        op::OpConfig::any cfg = op::OpConfig::any::object();
        cfg["bits"] = op::OpConfig::any(q.bits);
        cfg["group_size"] = op::OpConfig::any(q.group);
        cfg["zero_point"] = op::OpConfig::any(q.zp);
        cfg["has_zero_points"] = op::OpConfig::any(q.has_z);
        cfg["rms_norm"] = op::OpConfig::any(q.rms);
        cfg["rms_eps"] = op::OpConfig::any(q.eps);
        cfg["has_bias"] = op::OpConfig::any(q.has_bias);
        cfg["has_residual"] = op::OpConfig::any(q.has_res);
        cfg["act"] = op::OpConfig::any(std::string(q.gate ? "silu_gate" : "none"));
        return cfg;
    }

    // Rebuilds a graph node by node.  `replace` may emit a substitute for a node (returning what its output 0
    // maps to); everything else is re-created on the mapped inputs with the same operator object.
    class Rebuilder
    {
    public:
        explicit Rebuilder(const std::shared_ptr<Graph>& old_graph)
            : m_old(old_graph)
            , m_new(std::make_shared<Graph>())
        {
            for (auto& n : old_graph->get_ordered_ops())
                for (auto& e : n->get_in_edges())
                    m_users[e.src.get()].push_back(n);
        }
        const GNodeVector& users(const std::shared_ptr<GNode>& n) { return m_users[n.get()]; }
        bool single_user(const std::shared_ptr<GNode>& n) { return m_users[n.get()].size() == 1; }
        NodeOut map(const NodeOut& o) const
        {
            auto it = m_map.find({o.first.get(), o.second});
            NNFUSION_CHECK(it != m_map.end()) << "node " << o.first->get_name() << " used before it was rebuilt";
            return it->second;
        }
        std::shared_ptr<GNode> add(std::shared_ptr<op::Op> op, const std::vector<NodeOut>& inputs)
        {
            return m_new->add_node_and_edge(op, inputs);
        }
        std::shared_ptr<GNode> constant(const element::Type& elt, const Shape& shape, const void* data)
        {
            return m_new->add_node_and_edge(std::make_shared<op::Constant>(elt, shape, data), GNodeVector{});
        }
        using Replace = std::function<bool(const std::shared_ptr<GNode>&, Rebuilder&, std::vector<NodeOut>&)>;
        // runs the rebuild; returns the new graph without the nodes that no Result depends on
        std::shared_ptr<Graph> run(const Replace& replace)
        {
            for (auto& n : m_old->get_ordered_ops())
            {
                std::vector<NodeOut> outs;
                if (!replace(n, *this, outs))
                {
                    std::vector<NodeOut> ins;
                    for (size_t i = 0; i < n->get_input_size(); ++i)
                        ins.push_back(map(input_of(n, i)));
                    auto nn = add(n->get_op_ptr(), ins);
                    for (size_t i = 0; i < n->get_output_size(); ++i)
                        outs.push_back({nn, (int)i});
                }
                for (size_t i = 0; i < outs.size(); ++i)
                    m_map[{n.get(), (int)i}] = outs[i];
            }
            return prune(m_new);
        }

    private:
        static std::shared_ptr<Graph> prune(const std::shared_ptr<Graph>& g)
        {
            std::set<GNode*> live;
            const auto& nodes = g->get_ordered_ops();
            for (auto it = nodes.rbegin(); it != nodes.rend(); ++it)
            {
                if ((*it)->is_output() || (*it)->is_parameter() || live.count(it->get()))
                {
                    live.insert(it->get());
                    for (auto& e : (*it)->get_in_edges())
                        live.insert(e.src.get());
                }
            }
            if (live.size() == nodes.size())
                return g;
            auto out = std::make_shared<Graph>();
            std::map<GNode*, std::shared_ptr<GNode>> m;
            for (auto& n : nodes)
            {
                if (!live.count(n.get()))
                    continue;
                std::vector<NodeOut> ins;
                for (auto& e : n->get_in_edges())
                    ins.push_back({m.at(e.src.get()), e.src_output});
                m[n.get()] = out->add_node_and_edge(n->get_op_ptr(), ins);
            }
            return out;
        }

        std::shared_ptr<Graph> m_old, m_new;
        std::map<GNode*, GNodeVector> m_users;
        std::map<std::pair<GNode*, int>, NodeOut> m_map;
    };

    std::shared_ptr<op::Constant> constant_of(const NodeOut& o)
    {
        return std::dynamic_pointer_cast<op::Constant>(o.first->get_op_ptr());
    }
    // rows of several [n_i, cols] constants stacked into one [sum n_i, cols] constant
    std::shared_ptr<GNode> stack_rows(Rebuilder& rb, const std::vector<NodeOut>& parts)
    {
        const auto& first = parts[0].first;
        const Shape& s0 = first->get_output_shape(0);
        const element::Type& elt = first->get_output_element_type(0);
        size_t rows = 0;
        std::vector<uint8_t> data;
        for (auto& p : parts)
        {
            auto c = constant_of(p);
            NNFUSION_CHECK(c && p.first->get_output_shape(0).size() == 2 && p.first->get_output_shape(0)[1] == s0[1]);
            rows += p.first->get_output_shape(0)[0];
            data.insert(data.end(), c->get_data().begin(), c->get_data().end());
        }
        return rb.constant(elt, Shape{rows, s0[1]}, data.data());
    }

    bool same(const NodeOut& a, const NodeOut& b) { return a.first == b.first && a.second == b.second; }

    // SiLU(g): Swish(g) or Multiply(g, Sigmoid(g)) in either operand order; returns g's producer
    bool match_silu(const std::shared_ptr<GNode>& n, NodeOut& g)
    {
        if (is_op(n, "Swish"))
        {
            g = input_of(n, 0);
            return true;
        }
        if (!is_op(n, "Multiply"))
            return false;
        for (int k = 0; k < 2; ++k)
        {
            NodeOut x = input_of(n, k), sg = input_of(n, 1 - k);
            if (is_op(sg.first, "Sigmoid") && same(input_of(sg.first, 0), x))
            {
                g = x;
                return true;
            }
        }
        return false;
    }

    // every user of `n` is in `allowed`
    bool only_used_by(Rebuilder& rb, const std::shared_ptr<GNode>& n, std::initializer_list<std::shared_ptr<GNode>> allowed)
    {
        for (auto& u : rb.users(n))
        {
            bool ok = false;
            for (auto& a : allowed)
                ok = ok || a == u;
            if (!ok)
                return false;
        }
        return true;
    }

    // (z: the zero-point tensor as placed in the new graph; unused without one)
    std::vector<NodeOut> quant_dot_inputs(Rebuilder& rb, const QuantDotInfo& q, const NodeOut& wq, const NodeOut& s, const NodeOut& z)
    {
        std::vector<NodeOut> ins = {rb.map(q.a), wq, s};
        if (q.has_z)
            ins.push_back(z);
        if (q.rms)
            ins.push_back(rb.map(q.gamma));
        if (q.has_bias)
            ins.push_back(rb.map(q.bias));
        if (q.has_res)
            ins.push_back(rb.map(q.res));
        return ins;
    }

    // One sweep of the epilogue patterns; returns the number of rewrites.
    size_t fuse_epilogues_once(std::shared_ptr<Graph>& graph)
    {
        size_t count = 0;
        Rebuilder rb(graph);
        auto replace = [&](const std::shared_ptr<GNode>& n, Rebuilder& r, std::vector<NodeOut>& outs) -> bool {
            QuantDotInfo q;
            // (0) Dot{transpose_B}(A, Dequantize(Wq, S [, Z]))  ->  QuantDot(A, Wq, S [, Z]): the dequantised weights are
            // never written (precedent: the reference folds MatMul + Add into one node,
            // engine/pass/graph/subgraph_fusion_optimizer/matmuladd_fusion_optimizer.cpp)
            if (is_op(n, "Dot"))
            {
                auto& dcfg = generic(n)->localOpConfig.getRoot();
                NodeOut w = input_of(n, 1);
                if (!dcfg["transpose_B"].get<bool>() || dcfg["transpose_A"].get<bool>() || !is_op(w.first, "Dequantize"))
                    return false;
                auto& qcfg = generic(w.first)->localOpConfig.getRoot();
                QuantDotInfo f;
                f.bits = qcfg["bits"].get<int>();
                f.group = qcfg["group_size"].get<int>();
                f.zp = qcfg["zero_point"].get<int>();
                f.has_z = qcfg["has_zero_points"].get<bool>();
                f.a = input_of(n, 0);
                auto node = r.add(std::make_shared<op::GenericOp>(n->get_name(), "QuantDot", quant_dot_config(f)),
                                  quant_dot_inputs(r, f, r.map(input_of(w.first, 0)), r.map(input_of(w.first, 1)),
                                                   f.has_z ? r.map(input_of(w.first, 2)) : NodeOut()));
                outs = {{node, 0}};
                ++count;
                return true;
            }
            // (1) SiLU(QuantDot_gate(x)) * QuantDot_up(x)  ->  QuantDot{act = silu_gate} over [gate; up]
            if (is_op(n, "Multiply"))
            {
                for (int k = 0; k < 2; ++k)
                {
                    NodeOut silu = input_of(n, k), up = input_of(n, 1 - k), gate;
                    QuantDotInfo qg, qu;
                    if (!match_silu(silu.first, gate) || silu.first == n)
                        continue;
                    if (!quant_dot_info(gate.first, qg) || !quant_dot_info(up.first, qu) || gate.first == up.first)
                        continue;
                    if (qg.has_bias || qg.has_res || qg.gate || qu.has_bias || qu.has_res || qu.gate)
                        continue;
                    if (!same(qg.a, qu.a) || qg.rms != qu.rms || (qg.rms && (!same(qg.gamma, qu.gamma) || qg.eps != qu.eps)))
                        continue;
                    if (!qg.same_block_parameters(qu))
                        continue;
                    if (!constant_of(qg.wq) || !constant_of(qg.s) || !constant_of(qu.wq) || !constant_of(qu.s) ||
                        (qg.has_z && (!constant_of(qg.z) || !constant_of(qu.z))))
                        continue;
                    if (gate.first->get_output_shape(0) != up.first->get_output_shape(0))
                        continue;
                    // the gate feeds only the SiLU (and its sigmoid), the SiLU and the up projection only this product
                    bool gate_private = true;
                    for (auto& u : r.users(gate.first))
                        gate_private = gate_private && (u == silu.first || (is_op(u, "Sigmoid") && r.single_user(u) &&
                                                                            r.users(u)[0] == silu.first));
                    if (!gate_private || !only_used_by(r, silu.first, {n}) || !only_used_by(r, up.first, {n}))
                        continue;
                    auto wq = stack_rows(r, {qg.wq, qu.wq});
                    auto s = stack_rows(r, {qg.s, qu.s});
                    NodeOut z;
                    if (qg.has_z)
                        z = {stack_rows(r, {qg.z, qu.z}), 0};
                    QuantDotInfo f = qg;
                    f.gate = true;
                    auto node = r.add(std::make_shared<op::GenericOp>(n->get_name() + "_gate_up", "QuantDot", quant_dot_config(f)),
                                      quant_dot_inputs(r, f, {wq, 0}, {s, 0}, z));
                    outs = {{node, 0}};
                    ++count;
                    return true;
                }
                return false;
            }
            // (2) Add(QuantDot, bias constant [N]) / Add(QuantDot, residual [M,N])
            if (is_op(n, "Add"))
            {
                for (int k = 0; k < 2; ++k)
                {
                    NodeOut d = input_of(n, k), other = input_of(n, 1 - k);
                    if (!quant_dot_info(d.first, q) || q.gate || !r.single_user(d.first) || d.first == other.first)
                        continue;
                    const Shape& ys = d.first->get_output_shape(0);
                    const Shape& os = other.first->get_output_shape(other.second);
                    QuantDotInfo f = q;
                    if (!q.has_bias && !q.has_res && constant_of(other) && os.size() == 1 && os[0] == ys.back())
                    {
                        f.has_bias = true;
                        f.bias = other;
                    }
                    else if (!q.has_res && os == ys)
                    {
                        f.has_res = true;
                        f.res = other;
                    }
                    else
                        continue;
                    // the other operand must not depend on the QuantDot being rewritten: it is an earlier node or
                    // a constant, which the rebuild has already placed
                    auto node = r.add(std::make_shared<op::GenericOp>(d.first->get_name(), "QuantDot", quant_dot_config(f)),
                                      quant_dot_inputs(r, f, r.map(q.wq), r.map(q.s), q.has_z ? r.map(q.z) : NodeOut()));
                    outs = {{node, 0}};
                    ++count;
                    return true;
                }
                return false;
            }
            if (!quant_dot_info(n, q))
                return false;
            // (3) QuantDot(RMSNorm(x, gamma))  ->  QuantDot{rms_norm}(x, ..., gamma)
            if (!q.rms && is_op(q.a.first, "RMSNorm"))
            {
                QuantDotInfo f = q;
                f.rms = true;
                f.a = input_of(q.a.first, 0);
                f.gamma = input_of(q.a.first, 1);
                f.eps = generic(q.a.first)->localOpConfig.getRoot()["eps"].get<double>();
                auto node = r.add(std::make_shared<op::GenericOp>(n->get_name(), "QuantDot", quant_dot_config(f)),
                                  quant_dot_inputs(r, f, r.map(q.wq), r.map(q.s), q.has_z ? r.map(q.z) : NodeOut()));
                outs = {{node, 0}};
                ++count;
                return true;
            }
            // (4) down{residual = x}( gate_up{rms_norm, silu_gate}(x) )  ->  FusedQuantMLP
            QuantDotInfo gu;
            if (q.has_res && !q.has_bias && !q.rms && !q.gate && quant_dot_info(q.a.first, gu) && gu.rms && gu.gate &&
                !gu.has_bias && !gu.has_res && same(gu.a, q.res) && r.single_user(q.a.first) && gu.group == q.group &&
                gu.bits == q.bits && n->get_output_shape(0).size() == 2)
            {
                op::OpConfig::any cfg = op::OpConfig::any::object();
                cfg["bits"] = op::OpConfig::any(q.bits);
                cfg["group_size"] = op::OpConfig::any(q.group);
                cfg["zero_point"] = op::OpConfig::any(gu.zp);
                cfg["zero_point_down"] = op::OpConfig::any(q.zp);
                cfg["has_zero_points_gate_up"] = op::OpConfig::any(gu.has_z);
                cfg["has_zero_points_down"] = op::OpConfig::any(q.has_z);
                cfg["rms_eps"] = op::OpConfig::any(gu.eps);
                std::vector<NodeOut> ins = {r.map(gu.a), r.map(gu.gamma), r.map(gu.wq), r.map(gu.s), r.map(q.wq), r.map(q.s)};
                if (gu.has_z)
                    ins.push_back(r.map(gu.z));
                if (q.has_z)
                    ins.push_back(r.map(q.z));
                auto node = r.add(std::make_shared<op::GenericOp>(n->get_name() + "_mlp", "FusedQuantMLP", cfg), ins);
                outs = {{node, 0}};
                ++count;
                return true;
            }
            return false;
        };
        auto rebuilt = rb.run(replace);
        if (count)
            graph = rebuilt;
        return count;
    }
} // namespace

bool pass::graph::QuantEpilogueFusionPass::run_on_graph(std::shared_ptr<Graph>& graph)
{
    fused = 0;
    for (int sweep = 0; sweep < 16; ++sweep)
    {
        size_t c = fuse_epilogues_once(graph);
        fused += c;
        if (c == 0)
            break;
    }
    return true;
}

bool pass::graph::QuantGemmFusionPass::run_on_graph(std::shared_ptr<Graph>& graph)
{
    merged_groups = 0;
    // groups of mergeable QuantDots, keyed by what they read and how
    struct Group
    {
        std::vector<std::shared_ptr<GNode>> members;
    };
    std::vector<Group> groups;
    std::map<GNode*, size_t> group_of;
    {
        std::map<std::string, size_t> by_key;
        for (auto& n : graph->get_ordered_ops())
        {
            QuantDotInfo q;
            if (!quant_dot_info(n, q) || q.has_bias || q.has_res || q.gate || !constant_of(q.wq) || !constant_of(q.s) ||
                (q.has_z && !constant_of(q.z)))
                continue;
            std::ostringstream key;
            key << (void*)q.a.first.get() << ':' << q.a.second << '|' << q.rms << '|' << (void*)q.gamma.first.get() << '|' << q.eps
                << '|' << q.group << '|' << (q.has_z ? -1 : q.zp) << '|' << q.bits << '|' << q.wq.first->get_output_shape(0)[1];
            auto it = by_key.find(key.str());
            if (it == by_key.end())
            {
                by_key[key.str()] = groups.size();
                groups.push_back(Group());
                it = by_key.find(key.str());
            }
            groups[it->second].members.push_back(n);
        }
        for (size_t g = 0; g < groups.size(); ++g)
            if (groups[g].members.size() >= 2)
                for (auto& m : groups[g].members)
                    group_of[m.get()] = g;
    }
    if (group_of.empty())
        return true;
    std::map<size_t, std::vector<NodeOut>> slices; // group -> slice per member, made when the first member is reached
    Rebuilder rb(graph);
    auto replace = [&](const std::shared_ptr<GNode>& n, Rebuilder& r, std::vector<NodeOut>& outs) -> bool {
        auto it = group_of.find(n.get());
        if (it == group_of.end())
            return false;
        const Group& grp = groups[it->second];
        if (!slices.count(it->second))
        {
            std::vector<NodeOut> wqs, ss, zs;
            QuantDotInfo q0;
            quant_dot_info(grp.members[0], q0);
            for (auto& m : grp.members)
            {
                QuantDotInfo q;
                quant_dot_info(m, q);
                wqs.push_back(q.wq);
                ss.push_back(q.s);
                if (q.has_z)
                    zs.push_back(q.z);
            }
            auto wq = stack_rows(r, wqs);
            auto s = stack_rows(r, ss);
            NodeOut z;
            if (q0.has_z)
                z = {stack_rows(r, zs), 0};
            auto wide = r.add(std::make_shared<op::GenericOp>(grp.members[0]->get_name() + "_merged", "QuantDot", quant_dot_config(q0)),
                              quant_dot_inputs(r, q0, {wq, 0}, {s, 0}, z));
            int begin = 0;
            for (auto& m : grp.members)
            {
                const int rows = (int)m->get_output_shape(0).back();
                op::OpConfig::any cfg = op::OpConfig::any::object();
                cfg["begin"] = op::OpConfig::any(begin);
                cfg["end"] = op::OpConfig::any(begin + rows);
                slices[it->second].push_back({r.add(std::make_shared<op::GenericOp>(m->get_name() + "_slice", "Slice", cfg), {{wide, 0}}), 0});
                begin += rows;
            }
            ++merged_groups;
        }
        for (size_t i = 0; i < grp.members.size(); ++i)
            if (grp.members[i] == n)
                outs = {slices[it->second][i]};
        return true;
    };
    graph = rb.run(replace);
    return true;
}
