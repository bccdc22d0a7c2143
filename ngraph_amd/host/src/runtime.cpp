// Runtime plumbing: tensors, Executable validation, Backend::create, BackendManager's dlopen seam.
#include <dirent.h>
#include <dlfcn.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "ngraph/runtime/backend_manager.hpp"

using namespace std;

namespace ngraph
{
    namespace runtime
    {
        // ------------------------------------------------------------------ Tensor
        void Tensor::copy_from(const Tensor& source)
        {
            if (get_element_count() != source.get_element_count())
                throw invalid_argument("runtime::Tensor::copy_from: element count does not match");
            if (get_element_type() != source.get_element_type())
                throw invalid_argument("runtime::Tensor::copy_from: element types do not match");
            vector<uint8_t> bounce(get_size_in_bytes());
            source.read(bounce.data(), bounce.size());
            write(bounce.data(), bounce.size());
        }

        HostTensor::HostTensor(const element::Type& element_type, const Shape& shape, void* memory_pointer, const string& name)
            : Tensor(make_shared<descriptor::Tensor>(element_type, shape, name)), m_data(memory_pointer), m_owned(memory_pointer == nullptr)
        {
            if (m_owned)
            {
                size_t n = max<size_t>(get_size_in_bytes(), 1);
                if (posix_memalign(&m_data, 64, n) != 0)
                    throw bad_alloc();
            }
        }

        HostTensor::~HostTensor()
        {
            if (m_owned)
                free(m_data);
        }

        // whole-tensor transfers only (src/ngraph/runtime/host_tensor.cpp:147-185)
        void HostTensor::write(const void* p, size_t n)
        {
            if (n != get_size_in_bytes())
                throw out_of_range("partial tensor write not supported");
            if (n && !p)
                throw runtime_error("HostTensor::write: null source");
            if (n)
                memcpy(m_data, p, n);
        }

        void HostTensor::read(void* p, size_t n) const
        {
            if (n != get_size_in_bytes())
                throw out_of_range("partial tensor read access not supported");
            if (n && !p)
                throw runtime_error("HostTensor::read: null destination");
            if (n)
                memcpy(p, m_data, n);
        }

        // ------------------------------------------------------------------ Executable
        Executable::Executable() {}
        Executable::~Executable() {}

        bool Executable::call_with_validate(const vector<shared_ptr<Tensor>>& outputs, const vector<shared_ptr<Tensor>>& inputs)
        {
            validate(outputs, inputs);
            return call(outputs, inputs);
        }

        void Executable::validate(const vector<shared_ptr<Tensor>>& outputs, const vector<shared_ptr<Tensor>>& inputs)
        {
            const ParameterVector& parameters = get_parameters();
            const ResultVector& results = get_results();
            if (parameters.size() != inputs.size())
            {
                stringstream ss;
                ss << "Call input count " << inputs.size() << " does not match Function's Parameter count " << parameters.size();
                throw runtime_error(ss.str());
            }
            if (results.size() != outputs.size())
            {
                stringstream ss;
                ss << "Call output count " << outputs.size() << " does not match Function's Result count " << results.size();
                throw runtime_error(ss.str());
            }
            for (size_t i = 0; i < parameters.size(); i++)
            {
                if (parameters[i]->get_output_element_type(0) != inputs[i]->get_element_type())
                {
                    stringstream ss;
                    ss << "Input " << i << " type '" << inputs[i]->get_element_type() << "' does not match Parameter type '"
                       << parameters[i]->get_output_element_type(0) << "'";
                    throw runtime_error(ss.str());
                }
                if (parameters[i]->get_output_shape(0) != inputs[i]->get_shape())
                {
                    stringstream ss;
                    ss << "Input " << i << " shape " << inputs[i]->get_shape() << " does not match Parameter shape "
                       << parameters[i]->get_output_shape(0);
                    throw runtime_error(ss.str());
                }
            }
            for (size_t i = 0; i < results.size(); i++)
            {
                if (results[i]->get_output_element_type(0) != outputs[i]->get_element_type())
                {
                    stringstream ss;
                    ss << "Output " << i << " type '" << outputs[i]->get_element_type() << "' does not match Result type '"
                       << results[i]->get_output_element_type(0) << "'";
                    throw runtime_error(ss.str());
                }
                if (results[i]->get_output_shape(0) != outputs[i]->get_shape())
                {
                    stringstream ss;
                    ss << "Output " << i << " shape " << outputs[i]->get_shape() << " does not match max Result shape "
                       << results[i]->get_output_shape(0);
                    throw runtime_error(ss.str());
                }
            }
        }

        const ParameterVector& Executable::get_parameters() const { return m_parameters; }
        const ResultVector& Executable::get_results() const { return m_results; }
        size_t Executable::get_preferred_pipeline_depth() const { return 2; }
        void Executable::set_parameters_and_results(const Function& func)
        {
            m_parameters = func.get_parameters();
            m_results = func.get_results();
        }
        vector<PerformanceCounter> Executable::get_performance_data() const { return vector<PerformanceCounter>(); }
        void Executable::save(ostream&) { throw runtime_error("save operation unimplemented."); }
        shared_ptr<Tensor> Executable::create_input_tensor(size_t) { throw runtime_error("create_input_tensor unimplemented"); }
        shared_ptr<Tensor> Executable::create_input_tensor(size_t, void*) { throw runtime_error("create_input_tensor unimplemented"); }
        shared_ptr<Tensor> Executable::create_output_tensor(size_t) { throw runtime_error("create_output_tensor unimplemented"); }
        shared_ptr<Tensor> Executable::create_output_tensor(size_t, void*) { throw runtime_error("create_output_tensor unimplemented"); }
        vector<shared_ptr<Tensor>> Executable::create_input_tensor(size_t, size_t) { throw runtime_error("create_input_tensor unimplemented"); }
        vector<shared_ptr<Tensor>> Executable::create_output_tensor(size_t, size_t) { throw runtime_error("create_output_tensor unimplemented"); }

        // ------------------------------------------------------------------ Backend
        mutex Backend::m_mtx;
        string Backend::s_backend_shared_library_search_directory;

        Backend::~Backend() {}

        shared_ptr<Backend> Backend::create(const string& t, bool)
        {
            // "CPU_CODEGEN" style names: the first '_' separates name from options
            string type = t;
            auto pos = type.find('_');
            if (pos != string::npos)
                type = type.replace(pos, 1, ":");
            return BackendManager::create_backend(type);
        }

        vector<string> Backend::get_registered_devices() { return BackendManager::get_registered_backends(); }
        shared_ptr<Executable> Backend::compile(shared_ptr<Function> func, pass::PassConfig&, bool enable_performance_data)
        {
            return compile(func, enable_performance_data);
        }
        shared_ptr<Executable> Backend::load(istream&) { throw runtime_error("load operation unimplemented."); }
        bool Backend::is_supported(const Node&) const { return false; }
        bool Backend::is_supported_property(const Property) const { return false; }
        void Backend::remove_compiled_function(shared_ptr<Executable>) {}
        bool Backend::is_device_memory(void*) { return false; }

        void Backend::set_backend_shared_library_search_directory(const string& path)
        {
            lock_guard<mutex> lock(m_mtx);
            s_backend_shared_library_search_directory = path;
        }
        const string& Backend::get_backend_shared_library_search_directory()
        {
            if (s_backend_shared_library_search_directory.empty())
                s_backend_shared_library_search_directory = BackendManager::get_library_directory();
            return s_backend_shared_library_search_directory;
        }

        bool Backend::executable_can_create_tensors()
        {
            // probe with a trivial function, as src/ngraph/runtime/backend.cpp:154-173 does
            auto a = make_shared<op::v0::Parameter>(element::f32, Shape{});
            auto f = make_shared<Function>(OutputVector{Output<Node>(a, 0)}, ParameterVector{a});
            bool rc = true;
            try
            {
                auto exec = compile(f);
                exec->create_input_tensor(0);
                exec->create_output_tensor(0);
            }
            catch (...)
            {
                rc = false;
            }
            return rc;
        }

        // ------------------------------------------------------------------ BackendManager
        static string to_lower(string s)
        {
            transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return static_cast<char>(tolower(c)); });
            return s;
        }
        static string to_upper(string s)
        {
            transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return static_cast<char>(toupper(c)); });
            return s;
        }

        unordered_map<string, BackendConstructor>& BackendManager::get_registry()
        {
            static unordered_map<string, BackendConstructor> registry;
            return registry;
        }

        void BackendManager::register_backend(const string& name, BackendConstructor ctor) { get_registry()[name] = ctor; }

        string BackendManager::get_library_directory()
        {
            Dl_info info;
            if (dladdr(reinterpret_cast<void*>(&BackendManager::register_backend), &info) && info.dli_fname)
            {
                string path(info.dli_fname);
                auto slash = path.rfind('/');
                return slash == string::npos ? string(".") : path.substr(0, slash);
            }
            return ".";
        }

        void* BackendManager::open_shared_library(string type)
        {
            string name = "lib" + to_lower(type) + "_backend.so";
            string dir = Backend::get_backend_shared_library_search_directory();
            string path = dir.empty() ? name : dir + "/" + name;
            void* handle = dlopen(path.c_str(), RTLD_NOW | RTLD_GLOBAL);
            if (!handle)
            {
                stringstream ss;
                ss << "Unable to find backend '" << type << "' as file '" << path << "'\nOpen error message '" << dlerror() << "'";
                throw runtime_error(ss.str());
            }
            return handle;
        }

        shared_ptr<Backend> BackendManager::create_backend(string config)
        {
            string type = config, options;
            auto colon = type.find(':');
            if (colon != string::npos)
            {
                options = type.substr(colon + 1);
                type = type.substr(0, colon);
            }
            auto& registry = get_registry();
            auto it = registry.find(type);
            if (it == registry.end())
            {
                void* handle = open_shared_library(type);
                string sym = "ngraph_register_" + to_lower(type) + "_backend";
                auto register_plugin = reinterpret_cast<void (*)()>(dlsym(handle, sym.c_str()));
                if (!register_plugin)
                {
                    dlclose(handle);
                    throw runtime_error("Unable to find backend '" + type + "': shared library lacks symbol '" + sym + "'");
                }
                register_plugin();
                it = registry.find(type);
                if (it == registry.end())
                    throw runtime_error("Backend '" + type + "' not registered. Error:'");
            }
            return it->second(options);
        }

        vector<string> BackendManager::get_registered_backends()
        {
            vector<string> rc;
            for (const auto& p : get_registry())
                rc.push_back(p.first);
            // plus every lib*_backend.so next to this library
            string dir = Backend::get_backend_shared_library_search_directory();
            if (DIR* d = opendir(dir.c_str()))
            {
                while (dirent* e = readdir(d))
                {
                    string n = e->d_name;
                    const string pre = "lib", post = "_backend.so";
                    if (n.size() > pre.size() + post.size() && n.compare(0, pre.size(), pre) == 0 &&
                        n.compare(n.size() - post.size(), post.size(), post) == 0)
                    {
                        string name = to_upper(n.substr(pre.size(), n.size() - pre.size() - post.size()));
                        if (find(rc.begin(), rc.end(), name) == rc.end())
                            rc.push_back(name);
                    }
                }
                closedir(d);
            }
            return rc;
        }
    }
}
