// In-place annotations: which output may alias which input
// (src/nnfusion/core/operators/util/annotations.hpp:26-90).
#pragma once

#include "nnfusion/common/common.hpp"

namespace nnfusion
{
    namespace op
    {
        struct oi_pair
        {
            size_t output;
            size_t input;
            bool destructive;
            bool force_inplace = false;
            size_t input_offset = 0;
        };

        class Annotations
        {
        public:
            void add_in_place_oi_pair(const oi_pair& p) { m_pairs.push_back(p); }
            const std::vector<oi_pair>& get_in_place_oi_pairs() const { return m_pairs; }

        private:
            std::vector<oi_pair> m_pairs;
        };
    } // namespace op
    namespace kernels
    {
        using Annotations = op::Annotations;
    }
} // namespace nnfusion
