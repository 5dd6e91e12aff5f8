// op::Op and friends, graph::GNode / Graph, GenericOp / OpConfig.
#include "nnfusion/core/graph/gnode.hpp"
#include "nnfusion/core/operators/generic_op/generic_op.hpp"

#include <atomic>
#include <cstring>

namespace nnfusion
{
    namespace op
    {
        namespace
        {
            std::atomic<size_t> g_op_counter{0};
        }

        Op::Op(const std::string& op_type)
            : m_op_type(op_type)
        {
            m_unique_name = op_type + "_" + std::to_string(g_op_counter++);
        }

        void Parameter::validate_and_infer_types(std::shared_ptr<graph::GNode> gnode)
        {
            gnode->set_output_type_and_shape(0, m_elt, m_shape);
            gnode->get_output_tensor_ptr(0)->set_parameter();
        }

        Constant::Constant(const element::Type& elt, const Shape& shape, const void* data)
            : Op("Constant")
            , m_elt(elt)
            , m_shape(shape)
        {
            size_t bytes = shape_size(shape) * elt.size();
            m_data.resize(bytes);
            if (bytes)
            {
                NNFUSION_CHECK_NOT_NULLPTR(data);
                std::memcpy(m_data.data(), data, bytes);
            }
        }

        void Constant::validate_and_infer_types(std::shared_ptr<graph::GNode> gnode)
        {
            gnode->set_output_type_and_shape(0, m_elt, m_shape);
            gnode->get_output_tensor_ptr(0)->set_constant();
            gnode->get_output_tensor_ptr(0)->set_persistent();
        }

        void Result::validate_and_infer_types(std::shared_ptr<graph::GNode> gnode)
        {
            NNFUSION_CHECK(gnode->get_input_size() == 1) << "Result takes one input";
            gnode->set_output_type_and_shape(0, gnode->get_input_element_type(0), gnode->get_input_shape(0));
        }

        // ---- OpConfig registry ------------------------------------------------------------------
        std::unordered_map<std::string, OpConfig>& get_op_configs()
        {
            static std::unordered_map<std::string, OpConfig> configs;
            return configs;
        }

        OpConfig& build_op_config(const std::string& opname)
        {
            auto& configs = get_op_configs();
            NNFUSION_CHECK(configs.find(opname) == configs.end())
                << "OpConfig for opname `" << opname << "` is registered more than once.";
            configs[opname].attr("op", opname);
            return configs[opname];
        }

        OpConfig& lookup_op_config(const std::string& opname)
        {
            auto it = get_op_configs().find(opname);
            if (it != get_op_configs().end())
                return it->second;
            return build_op_config(opname);
        }

        std::string create_code_from_template(std::string templ, const OpConfig::any& feed_dict)
        {
            for (auto& kv : feed_dict.items())
            {
                std::string key = "@" + kv.first + "@";
                std::string value;
                switch (kv.second.kind())
                {
                case json_lite::String: value = kv.second.get<std::string>(); break;
                default: value = kv.second.dump(); break;
                }
                size_t pos = 0;
                while ((pos = templ.find(key, pos)) != std::string::npos)
                {
                    templ.replace(pos, key.size(), value);
                    pos += value.size();
                }
            }
            return templ;
        }

        GenericOp::GenericOp(const std::string& name, const std::string& opname, const OpConfig::any& customOpConfig)
            : Op(opname)
        {
            auto it = get_op_configs().find(opname);
            NNFUSION_CHECK(it != get_op_configs().end()) << "no OpConfig registered for `" << opname << "`";
            localOpConfig = it->second;
            set_name(name);
            // per-node attributes override the registered defaults
            if (customOpConfig.is_object())
                for (auto& kv : customOpConfig.items())
                    localOpConfig.getRoot()[kv.first] = kv.second;
            localOpConfig.check_constrait();
        }

        void GenericOp::validate_and_infer_types(std::shared_ptr<graph::GNode> gnode)
        {
            NNFUSION_CHECK(localOpConfig.f_infershape != nullptr)
                << "Not implemented infershape for Op: " << get_op_type();
            localOpConfig.check_constrait();
            localOpConfig.f_infershape(gnode);
        }
    } // namespace op

    namespace graph
    {
        GNode::GNode(std::shared_ptr<op::Op> op, const std::vector<std::shared_ptr<GNode>>& inputs)
            : m_op(op)
        {
            for (size_t i = 0; i < inputs.size(); ++i)
                m_in_edges.push_back(Edge{inputs[i], 0, (int)i});
            set_output_size(1);
        }

        void GNode::initialize() { m_op->validate_and_infer_types(shared_from_this()); }

        std::shared_ptr<descriptor::Tensor> GNode::get_input_tensor_ptr(size_t i) const
        {
            const Edge& e = m_in_edges.at(i);
            return e.src->get_output_tensor_ptr((size_t)e.src_output);
        }

        void GNode::set_output_size(size_t n)
        {
            while (m_outputs.size() < n)
            {
                std::string name = m_op->get_unique_name() + "_" + std::to_string(m_outputs.size());
                m_outputs.push_back(std::make_shared<descriptor::Tensor>(element::dynamic, Shape{}, name));
            }
            m_outputs.resize(n);
        }

        void GNode::set_output_type_and_shape(size_t i, const element::Type& elt, const Shape& shape)
        {
            if (i >= m_outputs.size())
                set_output_size(i + 1);
            m_outputs[i]->set_tensor_type(elt, shape);
        }

        std::shared_ptr<GNode> Graph::add_node_and_edge(std::shared_ptr<op::Op> op, const GNodeVector& inputs)
        {
            auto node = std::make_shared<GNode>(op, inputs);
            node->set_id((int64_t)m_nodes.size());
            node->initialize();
            m_nodes.push_back(node);
            return node;
        }

        std::shared_ptr<GNode>
            Graph::add_node_and_edge(std::shared_ptr<op::Op> op,
                                     const std::vector<std::pair<std::shared_ptr<GNode>, int>>& inputs)
        {
            GNodeVector srcs;
            for (auto& in : inputs)
                srcs.push_back(in.first);
            auto node = std::make_shared<GNode>(op, srcs);
            // re-point the edges at the requested outputs before inference
            auto& edges = const_cast<std::vector<Edge>&>(node->get_in_edges());
            for (size_t i = 0; i < inputs.size(); ++i)
                edges[i].src_output = inputs[i].second;
            node->set_id((int64_t)m_nodes.size());
            node->initialize();
            m_nodes.push_back(node);
            return node;
        }

        GNodeVector Graph::get_parameters() const
        {
            GNodeVector v;
            for (auto& n : m_nodes)
                if (n->is_parameter())
                    v.push_back(n);
            return v;
        }

        GNodeVector Graph::get_outputs() const
        {
            if (!m_outputs.empty())
                return m_outputs;
            GNodeVector v;
            for (auto& n : m_nodes)
                if (n->is_output())
                    v.push_back(n);
            return v;
        }
    } // namespace graph
} // namespace nnfusion
