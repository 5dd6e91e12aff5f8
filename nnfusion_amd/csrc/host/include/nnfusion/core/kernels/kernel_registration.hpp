// KernelRegistration / KernelRegistry / REGISTER_KERNEL_EMITTER: static registration of emitters and
// lookup by (op, device, data type) (src/nnfusion/core/kernels/kernel_registration.hpp:13-122, .cpp:8-114).
#pragma once

#include "nnfusion/core/kernels/kernel_emitter.hpp"

namespace nnfusion
{
    namespace kernels
    {
        class KernelRegistration
        {
        public:
            typedef std::shared_ptr<KernelEmitter> (*Factory)(std::shared_ptr<KernelContext>);
            explicit KernelRegistration(const std::string op_name)
                : m_op_name(op_name)
            {
            }
            KernelRegistration& Device(const NNFusion_DeviceType device_type)
            {
                m_device_type = device_type;
                return *this;
            }
            KernelRegistration& TypeConstraint(const element::Type data_type)
            {
                m_data_type = data_type;
                return *this;
            }
            KernelRegistration& Tag(const std::string tag)
            {
                m_tag = tag;
                return *this;
            }
            KernelRegistration& Priority(size_t priority)
            {
                m_priority = priority;
                return *this;
            }
            KernelRegistration& KernelFactory(const Factory factory)
            {
                m_factory = factory;
                return *this;
            }
            // checks the required fields and hands the registration over
            const std::shared_ptr<KernelRegistration> Build();
            const std::string op_name() { return m_op_name; }
            void set_priority(size_t priority) { m_priority = priority; }

            std::string m_op_name;
            NNFusion_DeviceType m_device_type = UNKNOWN;
            element::Type m_data_type;
            std::string m_tag;
            Factory m_factory = nullptr;
            size_t m_priority = 0;
        };

        // start of the builder chain: Name("Op").Device(..).TypeConstraint(..).Tag(..).Priority(..)
        KernelRegistration& Name(const std::string op_name);

        class KernelRegistry
        {
        public:
            bool RegisterKernel(const std::string op_name, std::shared_ptr<KernelRegistration> registration);
            // the first / all registrations of op_name whose device and data type match
            std::shared_ptr<const KernelRegistration>
                FindKernelRegistration(const std::string op_name, const NNFusion_DeviceType& device_type,
                                       const element::Type data_type);
            std::vector<std::shared_ptr<const KernelRegistration>>
                FindKernelRegistrations(const std::string op_name, const NNFusion_DeviceType& device_type,
                                        const element::Type data_type);
            // highest priority among matched registrations
            std::shared_ptr<const KernelRegistration>
                KernelSelect(std::vector<std::shared_ptr<const KernelRegistration>>& matched_regs);
            size_t RegisteredKernelSize() const { return m_kernel_registry.size(); }
            static KernelRegistry* Global();

        private:
            std::unordered_multimap<std::string, std::shared_ptr<KernelRegistration>> m_kernel_registry;
        };

        class KernelRegistrar
        {
        public:
            KernelRegistrar(const std::string op_name, std::shared_ptr<KernelRegistration> registration)
            {
                KernelRegistry::Global()->RegisterKernel(op_name, registration);
            }
        };

#define NNF_CONCAT_IMPL(x, y) x##y
#define NNF_CONCAT(x, y) NNF_CONCAT_IMPL(x, y)

#define REGISTER_KERNEL_EMITTER(op_name, attrs, constructor)                                                   \
    static ::nnfusion::kernels::KernelRegistrar NNF_CONCAT(kernel_registrar, __COUNTER__)(                      \
        op_name,                                                                                               \
        ::nnfusion::kernels::Name(op_name)                                                                     \
            .attrs                                                                                             \
            .KernelFactory([](std::shared_ptr<::nnfusion::kernels::KernelContext> context)                     \
                               -> std::shared_ptr<::nnfusion::kernels::KernelEmitter> {                        \
                return std::make_shared<constructor>(context);                                                 \
            })                                                                                                 \
            .Build());
    } // namespace kernels
} // namespace nnfusion
