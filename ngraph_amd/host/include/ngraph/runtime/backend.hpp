// runtime::Backend: the plugin interface a device implements.
// Mirrors src/ngraph/runtime/backend.hpp:43-184 and backend.cpp:38-173 of the nGraph tree.
#pragma once

#include <istream>
#include <mutex>

#include "ngraph/pass.hpp"
#include "ngraph/runtime/executable.hpp"

namespace ngraph
{
    namespace runtime
    {
        class NGRAPH_API Backend
        {
        public:
            virtual ~Backend();
            // "NAME" or "NAME:options"; the first '_' of the name is read as ':' ("CPU_CODEGEN").
            // Throws std::runtime_error for an unknown backend.
            static std::shared_ptr<Backend> create(const std::string& type, bool must_support_dynamic = false);
            static std::vector<std::string> get_registered_devices();

            virtual std::shared_ptr<Tensor> create_tensor() = 0;
            virtual std::shared_ptr<Tensor> create_tensor(const element::Type& element_type, const Shape& shape) = 0;
            // memory_pointer is caller-owned and must outlive the tensor
            virtual std::shared_ptr<Tensor> create_tensor(const element::Type& element_type, const Shape& shape, void* memory_pointer) = 0;
            template <typename T>
            std::shared_ptr<Tensor> create_tensor(const Shape& shape)
            {
                return create_tensor(element::from<T>(), shape);
            }
            virtual bool supports_dynamic_tensors() { return false; }
            virtual std::shared_ptr<Executable> compile(std::shared_ptr<Function> func, bool enable_performance_data = false) = 0;
            virtual std::shared_ptr<Executable> compile(std::shared_ptr<Function> func, pass::PassConfig& pass_config, bool enable_performance_data = false);
            virtual std::shared_ptr<Executable> load(std::istream& input_stream);
            virtual bool is_supported(const Node& node) const;
            enum class Property
            {
                memory_attach
            };
            virtual bool is_supported_property(const Property prop) const;
            virtual void remove_compiled_function(std::shared_ptr<Executable> exec);
            static void set_backend_shared_library_search_directory(const std::string& path);
            static const std::string& get_backend_shared_library_search_directory();
            virtual bool is_device_memory(void* ptr);
            virtual bool executable_can_create_tensors();
            virtual std::string get_version() const { return "0.0.0"; }

        private:
            static std::mutex m_mtx;
            static std::string s_backend_shared_library_search_directory;
        };
    }
}
