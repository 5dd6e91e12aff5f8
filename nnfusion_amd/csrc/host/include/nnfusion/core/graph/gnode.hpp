// graph::GNode / graph::Graph: the slice of the graph IR that kernel selection, emitters and codegen
// touch (src/nnfusion/core/graph/gnode.hpp:77-172, graph.hpp:40-122, src/nnfusion/core/IR/attribute.hpp:226-302
// for the tag map).
#pragma once

#include "nnfusion/common/descriptor/tensor.hpp"
#include "nnfusion/core/operators/op.hpp"

namespace nnfusion
{
    namespace graph
    {
        // One tag: a type-erased value.  (*gnode)["Key"] = v;  (*gnode)["Key"].is_valid();  .as<T>()
        class Tag
        {
        public:
            bool is_valid() const { return (bool)m_value; }
            template <typename T>
            T& as()
            {
                NNFUSION_CHECK(m_value && m_type == &typeid(T)) << "tag is unset or holds another type";
                return *static_cast<T*>(m_value.get());
            }
            template <typename T>
            Tag& operator=(const T& v)
            {
                m_value = std::shared_ptr<void>(new T(v), [](void* p) { delete static_cast<T*>(p); });
                m_type = &typeid(T);
                return *this;
            }
            void reset()
            {
                m_value.reset();
                m_type = nullptr;
            }

        private:
            std::shared_ptr<void> m_value;
            const std::type_info* m_type = nullptr;
        };

        class Tagable
        {
        public:
            Tag& operator[](const std::string& key) { return m_tags[key]; }
            template <typename T>
            void Set(const std::string& key, const T& v)
            {
                m_tags[key] = v;
            }

        private:
            std::unordered_map<std::string, Tag> m_tags;
        };

        class GNode;
        struct Edge
        {
            std::shared_ptr<GNode> src;
            int src_output;
            int dst_input;
            std::shared_ptr<GNode> get_src() const { return src; }
            int get_src_output() const { return src_output; }
            int get_dst_input() const { return dst_input; }
        };

        class GNode : public Tagable, public std::enable_shared_from_this<GNode>
        {
        public:
            GNode(std::shared_ptr<op::Op> op, const std::vector<std::shared_ptr<GNode>>& inputs);
            // called once by Graph::add_node_and_edge after construction (needs shared_from_this)
            void initialize();

            const std::string& get_op_type() const { return m_op->get_op_type(); }
            std::shared_ptr<op::Op> get_op_ptr() const { return m_op; }
            const std::string& get_name() const { return m_op->get_name(); }
            const std::string& get_unique_name() const { return m_op->get_unique_name(); }
            size_t get_input_size() const { return m_in_edges.size(); }
            size_t get_output_size() const { return m_outputs.size(); }
            std::shared_ptr<descriptor::Tensor> get_input_tensor_ptr(size_t i) const;
            std::shared_ptr<descriptor::Tensor> get_output_tensor_ptr(size_t i) const { return m_outputs.at(i); }
            const Shape& get_input_shape(size_t i) const { return get_input_tensor_ptr(i)->get_shape(); }
            const Shape& get_output_shape(size_t i) const { return m_outputs.at(i)->get_shape(); }
            const Shape& get_shape() const { return get_output_shape(0); }
            const element::Type& get_input_element_type(size_t i) const { return get_input_tensor_ptr(i)->get_element_type(); }
            const element::Type& get_output_element_type(size_t i) const { return m_outputs.at(i)->get_element_type(); }
            const element::Type& get_element_type() const { return get_output_element_type(0); }
            void set_output_size(size_t n);
            void set_output_type_and_shape(size_t i, const element::Type& elt, const Shape& shape);
            const Edge& get_in_edge(size_t i) const { return m_in_edges.at(i); }
            const std::vector<Edge>& get_in_edges() const { return m_in_edges; }
            bool is_constant() const { return m_op->is_constant(); }
            bool is_parameter() const { return m_op->is_parameter(); }
            bool is_output() const { return m_op->is_output(); }
            int64_t get_id() const { return m_id; }
            void set_id(int64_t id) { m_id = id; }

        private:
            std::shared_ptr<op::Op> m_op;
            std::vector<Edge> m_in_edges;
            std::vector<std::shared_ptr<descriptor::Tensor>> m_outputs;
            int64_t m_id = -1;
        };
        using GNodeVector = std::vector<std::shared_ptr<GNode>>;

        class Graph
        {
        public:
            // creates the node, wires it to `inputs` (output 0 of each) and runs shape inference
            std::shared_ptr<GNode> add_node_and_edge(std::shared_ptr<op::Op> op, const GNodeVector& inputs);
            // inputs given as (node, output index) pairs
            std::shared_ptr<GNode> add_node_and_edge(std::shared_ptr<op::Op> op,
                                                     const std::vector<std::pair<std::shared_ptr<GNode>, int>>& inputs);
            const GNodeVector& get_nodes() const { return m_nodes; }
            // nodes are kept in insertion order, which is a topological order by construction
            const GNodeVector& get_ordered_ops() const { return m_nodes; }
            GNodeVector get_parameters() const;
            GNodeVector get_outputs() const;
            void set_outputs(const GNodeVector& outs) { m_outputs = outs; }

        private:
            GNodeVector m_nodes;
            GNodeVector m_outputs;
        };
    } // namespace graph
} // namespace nnfusion
