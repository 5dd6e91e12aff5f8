// descriptor::Tensor: what an emitter knows about a tensor (src/nnfusion/common/descriptor/tensor.hpp:40-118).
#pragma once

#include "nnfusion/common/type/element_type.hpp"

namespace nnfusion
{
    namespace descriptor
    {
        class Tensor
        {
        public:
            Tensor(const element::Type& elt, const PartialShape& shape, const std::string& name,
                   NNFusion_DeviceType device = UNKNOWN, bool is_persistent = false, bool is_constant = false,
                   bool is_parameter = false, bool is_RDMA_tensor = false, const std::string& group = "",
                   int device_id = -1)
                : m_elt(elt)
                , m_shape(shape)
                , m_name(name)
                , m_device(device)
                , m_persistent(is_persistent)
                , m_constant(is_constant)
                , m_parameter(is_parameter)
                , m_rdma(is_RDMA_tensor)
                , m_group(group)
                , m_device_id(device_id)
            {
            }
            const std::string& get_name() const { return m_name; }
            void set_name(const std::string& n) { m_name = n; }
            const element::Type& get_element_type() const { return m_elt; }
            const Shape& get_shape() const { return m_shape; }
            void set_tensor_type(const element::Type& elt, const PartialShape& shape)
            {
                m_elt = elt;
                m_shape = shape;
            }
            // bytes (in_byte) or elements
            size_t size(bool in_byte = true) const { return shape_size(m_shape) * (in_byte ? m_elt.size() : 1); }
            bool is_persistent() const { return m_persistent; }
            bool is_constant() const { return m_constant; }
            bool is_parameter() const { return m_parameter; }
            bool is_RDMA_tensor() const { return m_rdma; }
            void set_persistent(bool v = true) { m_persistent = v; }
            void set_constant(bool v = true) { m_constant = v; }
            void set_parameter(bool v = true) { m_parameter = v; }
            NNFusion_DeviceType get_device_type() const { return m_device; }
            void set_device_type(NNFusion_DeviceType d) { m_device = d; }
            int get_device_id() const { return m_device_id; }
            const std::string& get_group() const { return m_group; }
            void set_pool_offset(size_t off) { m_pool_offset = off; }
            size_t get_pool_offset() const { return m_pool_offset; }
            void set_pool(const std::string& p) { m_pool = p; }
            const std::string& get_pool() const { return m_pool; }
            void set_memset(bool flag, int value)
            {
                m_memset = flag;
                m_memset_value = value;
            }
            bool is_memset() const { return m_memset; }
            int get_memset_value() const { return m_memset_value; }

        private:
            element::Type m_elt;
            Shape m_shape;
            std::string m_name;
            NNFusion_DeviceType m_device;
            bool m_persistent, m_constant, m_parameter, m_rdma;
            std::string m_group;
            int m_device_id;
            size_t m_pool_offset = SIZE_MAX;
            std::string m_pool;
            bool m_memset = false;
            int m_memset_value = 0;
        };
    } // namespace descriptor
} // namespace nnfusion
