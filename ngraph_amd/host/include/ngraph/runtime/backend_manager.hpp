// runtime::BackendManager: registry of backend constructors and loader of lib<name>_backend.so.
// Mirrors src/ngraph/runtime/backend_manager.hpp:41-57 and backend_manager.cpp:51-229.
#pragma once

#include <functional>
#include <unordered_map>

#include "ngraph/runtime/backend.hpp"

namespace ngraph
{
    namespace runtime
    {
        using BackendConstructor = std::function<std::shared_ptr<Backend>(const std::string& config)>;

        class NGRAPH_API BackendManager
        {
            friend class Backend;

        public:
            // called by a plugin's ngraph_register_<name>_backend()
            static void register_backend(const std::string& name, BackendConstructor backend_constructor);
            static std::vector<std::string> get_registered_backends();

        private:
            static std::shared_ptr<Backend> create_backend(std::string type);
            static std::unordered_map<std::string, BackendConstructor>& get_registry();
            static void* open_shared_library(std::string type);
            static std::string get_library_directory();
        };
    }
}
