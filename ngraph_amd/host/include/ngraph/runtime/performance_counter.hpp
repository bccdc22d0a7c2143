// Per-op timing record returned by Executable::get_performance_data().
// Mirrors src/ngraph/runtime/performance_counter.hpp:28-46 of the nGraph tree.
#pragma once

#include "ngraph/core.hpp"

namespace ngraph
{
    namespace runtime
    {
        class NGRAPH_API PerformanceCounter
        {
        public:
            PerformanceCounter(const std::shared_ptr<const Node>& n, size_t us, size_t calls)
                : m_node(n), m_total_microseconds(us), m_call_count(calls)
            {
            }
            std::shared_ptr<const Node> get_node() const { return m_node; }
            size_t total_microseconds() const { return m_total_microseconds; }
            size_t microseconds() const { return m_call_count == 0 ? 0 : m_total_microseconds / m_call_count; }
            size_t call_count() const { return m_call_count; }

        private:
            std::shared_ptr<const Node> m_node;
            size_t m_total_microseconds;
            size_t m_call_count;
        };
    }
}
