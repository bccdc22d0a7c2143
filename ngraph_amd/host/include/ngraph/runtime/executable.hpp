// runtime::Executable: a compiled Function.
// Mirrors src/ngraph/runtime/executable.hpp:19-162 and executable.cpp:32-129 of the nGraph tree.
#pragma once

#include <ostream>

#include "ngraph/ops.hpp"
#include "ngraph/runtime/performance_counter.hpp"
#include "ngraph/runtime/tensor.hpp"

namespace ngraph
{
    namespace runtime
    {
        class NGRAPH_API Executable
        {
        public:
            Executable();
            virtual ~Executable();
            // returns true on success; errors are exceptions
            virtual bool call(const std::vector<std::shared_ptr<Tensor>>& outputs, const std::vector<std::shared_ptr<Tensor>>& inputs) = 0;
            bool call_with_validate(const std::vector<std::shared_ptr<Tensor>>& outputs, const std::vector<std::shared_ptr<Tensor>>& inputs);
            // throws std::runtime_error on a count / element type / shape mismatch
            void validate(const std::vector<std::shared_ptr<Tensor>>& outputs, const std::vector<std::shared_ptr<Tensor>>& inputs);
            virtual std::vector<PerformanceCounter> get_performance_data() const;
            const ParameterVector& get_parameters() const;
            const ResultVector& get_results() const;
            virtual size_t get_preferred_pipeline_depth() const;
            virtual void save(std::ostream& output_stream);
            virtual std::shared_ptr<Tensor> create_input_tensor(size_t input_index);
            virtual std::shared_ptr<Tensor> create_input_tensor(size_t input_index, void* memory_pointer);
            virtual std::shared_ptr<Tensor> create_output_tensor(size_t output_index);
            virtual std::shared_ptr<Tensor> create_output_tensor(size_t output_index, void* memory_pointer);
            virtual std::vector<std::shared_ptr<Tensor>> create_input_tensor(size_t input_index, size_t pipeline_depth);
            virtual std::vector<std::shared_ptr<Tensor>> create_output_tensor(size_t output_index, size_t pipeline_depth);

        protected:
            // must be called at the end of compile(), or validate() sees empty vectors
            void set_parameters_and_results(const Function& func);
            ParameterVector m_parameters;
            ResultVector m_results;
        };
    }
}
