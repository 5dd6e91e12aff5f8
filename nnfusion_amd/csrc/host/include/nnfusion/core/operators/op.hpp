// op::Op: base class of graph operators (src/nnfusion/core/operators/op.hpp:63-140).
#pragma once

#include "nnfusion/common/common.hpp"
#include "nnfusion/common/type/element_type.hpp"
#include "nnfusion/core/operators/util/annotations.hpp"

namespace nnfusion
{
    namespace graph
    {
        class GNode;
    }
    namespace op
    {
        class Op
        {
        public:
            explicit Op(const std::string& op_type);
            virtual ~Op() = default;
            const std::string& get_op_type() const { return m_op_type; }
            const std::string& get_name() const { return m_name.empty() ? m_unique_name : m_name; }
            void set_name(const std::string& n) { m_name = n; }
            const std::string& get_unique_name() const { return m_unique_name; }
            virtual void validate_and_infer_types(std::shared_ptr<graph::GNode> gnode) { (void)gnode; }
            virtual bool is_parameter() const { return false; }
            virtual bool is_output() const { return false; }
            virtual bool is_constant() const { return false; }
            virtual bool is_variable() const { return false; }
            virtual bool is_tensor_op() const { return is_parameter() || is_constant() || is_variable(); }
            std::shared_ptr<Annotations> get_op_annotations() const { return m_annotations; }
            void set_op_annotations(std::shared_ptr<Annotations> a) { m_annotations = a; }

        protected:
            std::string m_op_type;
            std::string m_name;
            std::string m_unique_name; // <op_type>_<instance counter>
            std::shared_ptr<Annotations> m_annotations;
        };

        // graph inputs, constants and outputs (op_define/{parameter,constant,result}.hpp in the tree)
        class Parameter : public Op
        {
        public:
            Parameter(const element::Type& elt, const Shape& shape)
                : Op("Parameter")
                , m_elt(elt)
                , m_shape(shape)
            {
            }
            bool is_parameter() const override { return true; }
            void validate_and_infer_types(std::shared_ptr<graph::GNode> gnode) override;

        private:
            element::Type m_elt;
            Shape m_shape;
        };

        class Constant : public Op
        {
        public:
            // data: raw bytes of the tensor (shape_size * elt.size())
            Constant(const element::Type& elt, const Shape& shape, const void* data);
            bool is_constant() const override { return true; }
            void validate_and_infer_types(std::shared_ptr<graph::GNode> gnode) override;
            const std::vector<uint8_t>& get_data() const { return m_data; }
            const void* get_data_ptr() const { return m_data.data(); }
            size_t get_data_size() const { return m_data.size(); }

        private:
            element::Type m_elt;
            Shape m_shape;
            std::vector<uint8_t> m_data;
        };

        class Result : public Op
        {
        public:
            Result()
                : Op("Result")
            {
            }
            bool is_output() const override { return true; }
            void validate_and_infer_types(std::shared_ptr<graph::GNode> gnode) override;
        };
    } // namespace op
} // namespace nnfusion
