// nbench: benchmark a serialized nGraph model on a backend.
//
// Command line, data initialisation and timing protocol follow nGraph's tool of the same name:
//   options            src/tools/nbench/nbench.cpp:157-253 (-f -b -d -i -w -s --timing_detail
//                      --no_copy_data --dump_results; the Graphviz options and --double_buffer are
//                      recognised and refused)
//   run_benchmark      src/tools/nbench/benchmark.cpp:87-185: compile once, one tensor per Parameter
//                      filled by random_init, `warmup_iterations` untimed then `iterations` timed
//                      calls on a wall clock; unless --no_copy_data every stale argument is written
//                      before and every result read after each call; "<ms>ms per iteration"
//   random_init        src/tools/nbench/benchmark_utils.cpp:30-117: reals uniform in [-1, 1), i8 in
//                      {-1, 0, 1}, other integers in {0, 1}, one unseeded default_random_engine
//   per-op timings     print_results / print_times, nbench.cpp:48-155 (plain ms columns here)
#include <algorithm>
#include <chrono>
#include <cstring>
#include <dirent.h>
#include <iomanip>
#include <iostream>
#include <map>
#include <random>
#include <set>
#include <sstream>
#include <sys/stat.h>

#include "ngraph/ngraph.hpp"
#include "ngraph/runtime/host_tensor.hpp"
#include "ngraph/serializer.hpp"

using namespace std;
using namespace ngraph;

namespace
{
    default_random_engine& get_random_engine()
    {
        static default_random_engine engine;
        return engine;
    }

    template <typename T>
    void init_int_tensor(runtime::HostTensor& t, int lo, int hi)
    {
        uniform_int_distribution<int> dist(lo, hi);
        T* p = t.get_data_ptr<T>();
        for (size_t i = 0; i < t.get_element_count(); ++i)
            p[i] = static_cast<T>(dist(get_random_engine()));
    }

    template <typename T>
    void init_real_tensor(runtime::HostTensor& t, T lo, T hi)
    {
        uniform_real_distribution<T> dist(lo, hi);
        T* p = t.get_data_ptr<T>();
        for (size_t i = 0; i < t.get_element_count(); ++i)
            p[i] = dist(get_random_engine());
    }

    void random_init(runtime::HostTensor& t)
    {
        switch (t.get_element_type().get_type_enum())
        {
        case element::Type_t::boolean: init_int_tensor<char>(t, 0, 1); break;
        case element::Type_t::f32: init_real_tensor<float>(t, -1, 1); break;
        case element::Type_t::f64: init_real_tensor<double>(t, -1, 1); break;
        case element::Type_t::i8: init_int_tensor<int8_t>(t, -1, 1); break;
        case element::Type_t::i32: init_int_tensor<int32_t>(t, 0, 1); break;
        case element::Type_t::i64: init_int_tensor<int64_t>(t, 0, 1); break;
        case element::Type_t::u8: init_int_tensor<uint8_t>(t, 0, 1); break;
        default: throw runtime_error("unsupported type");
        }
    }

    class stopwatch
    {
    public:
        void start() { m_start = chrono::steady_clock::now(); }
        void stop() { m_stop = chrono::steady_clock::now(); }
        double get_milliseconds() const { return chrono::duration<double, milli>(m_stop - m_start).count(); }
        double elapsed_milliseconds() const { return chrono::duration<double, milli>(chrono::steady_clock::now() - m_start).count(); }

    private:
        chrono::steady_clock::time_point m_start, m_stop;
    };

    template <typename T>
    void dump_elements(const runtime::HostTensor& t)
    {
        const T* p = static_cast<const T*>(t.get_data_ptr());
        cout << "[ ";
        for (size_t i = 0; i < t.get_element_count(); ++i)
            cout << +p[i] << " ";
        cout << "]";
    }

    void dump_result_tensors(const vector<shared_ptr<runtime::HostTensor>>& results)
    {
        size_t i = 0;
        for (const auto& r : results)
        {
            cout << "\nResult " << i++ << " (" << r->get_element_type() << " " << r->get_shape() << "): ";
            switch (r->get_element_type().get_type_enum())
            {
            case element::Type_t::f32: dump_elements<float>(*r); break;
            case element::Type_t::f64: dump_elements<double>(*r); break;
            case element::Type_t::i8: dump_elements<int8_t>(*r); break;
            case element::Type_t::u8: dump_elements<uint8_t>(*r); break;
            case element::Type_t::i32: dump_elements<int32_t>(*r); break;
            case element::Type_t::i64: dump_elements<int64_t>(*r); break;
            case element::Type_t::boolean: dump_elements<char>(*r); break;
            default: throw runtime_error("unsupported type");
            }
            cout << "\n";
        }
    }

    vector<runtime::PerformanceCounter> run_benchmark(const shared_ptr<Function>& f,
                                                      const string& backend_name,
                                                      size_t iterations,
                                                      bool timing_detail,
                                                      size_t warmup_iterations,
                                                      bool copy_data,
                                                      bool dump_results)
    {
        stopwatch timer;
        timer.start();
        auto backend = runtime::Backend::create(backend_name);
        auto exec = backend->compile(f, timing_detail);
        timer.stop();
        cout << "compile time: " << timer.get_milliseconds() << "ms" << endl;

        vector<shared_ptr<runtime::HostTensor>> arg_data;
        vector<shared_ptr<runtime::Tensor>> args;
        for (const auto& param : f->get_parameters())
        {
            auto tensor = backend->create_tensor(param->get_element_type(), param->get_output_shape(0));
            auto data = make_shared<runtime::HostTensor>(param->get_element_type(), param->get_output_shape(0));
            random_init(*data);
            tensor->write(data->get_data_ptr(), data->get_size_in_bytes());
            args.push_back(tensor);
            arg_data.push_back(data);
        }
        vector<shared_ptr<runtime::HostTensor>> result_data;
        vector<shared_ptr<runtime::Tensor>> results;
        for (const auto& out : f->get_results())
        {
            results.push_back(backend->create_tensor(out->get_output_element_type(0), out->get_output_shape(0)));
            result_data.push_back(make_shared<runtime::HostTensor>(out->get_output_element_type(0), out->get_output_shape(0)));
        }

        stopwatch t1;
        t1.start(); // restarted after the warm-up; started here so that zero iterations still reads a clock
        for (size_t i = 0; i < iterations + warmup_iterations; i++)
        {
            if (i == warmup_iterations)
                t1.start();
            if (copy_data)
                for (size_t a = 0; a < args.size(); a++)
                    if (args[a]->get_stale())
                        args[a]->write(arg_data[a]->get_data_ptr(), arg_data[a]->get_size_in_bytes());
            exec->call(results, args);
            if (copy_data)
                for (size_t r = 0; r < results.size(); r++)
                    results[r]->read(result_data[r]->get_data_ptr(), result_data[r]->get_size_in_bytes());
        }
        t1.stop();
        cout << t1.get_milliseconds() / static_cast<double>(iterations ? iterations : 1) << "ms per iteration" << endl;

        if (dump_results)
        {
            if (!copy_data) // nothing was read back inside the loop
                for (size_t r = 0; r < results.size(); r++)
                    results[r]->read(result_data[r]->get_data_ptr(), result_data[r]->get_size_in_bytes());
            dump_result_tensors(result_data);
        }
        return exec->get_performance_data();
    }

    string shape_text(const Shape& s)
    {
        ostringstream ss;
        ss << "{";
        for (size_t i = 0; i < s.size(); ++i)
            ss << (i ? "," : "") << s[i];
        ss << "}";
        return ss.str();
    }

    void print_times(const multimap<size_t, string>& timing)
    {
        size_t name_width = 0;
        for (const auto& p : timing)
            name_width = max(name_width, p.second.size());
        for (auto it = timing.rbegin(); it != timing.rend(); ++it)
            cout << setw(static_cast<int>(name_width + 2)) << left << it->second << setw(12) << right << fixed << setprecision(3)
                 << static_cast<double>(it->first) / 1000.0 << "ms\n";
    }

    void print_results(const vector<runtime::PerformanceCounter>& perf_data, bool timing_detail)
    {
        map<string, size_t> per_type, per_shape;
        multimap<size_t, string> per_node;
        for (const auto& p : perf_data)
        {
            auto node = p.get_node();
            string type = node->description();
            per_type[type] += p.microseconds();
            string key = type + shape_text(node->get_output_shape(0));
            per_shape[key] += p.microseconds();
            per_node.insert({p.microseconds(), node->get_name() + " " + key});
        }
        multimap<size_t, string> by_type, by_shape;
        for (const auto& t : per_type)
            by_type.insert({t.second, t.first});
        for (const auto& t : per_shape)
            by_shape.insert({t.second, t.first});
        if (by_type.empty())
            return;
        cout << "\n---- Aggregate times per op type ----\n";
        print_times(by_type);
        cout << "\n---- Aggregate times per op type/shape ----\n";
        print_times(by_shape);
        if (timing_detail)
        {
            cout << "\n---- Times per op ----\n";
            print_times(per_node);
        }
    }

    void print_statistics(const shared_ptr<Function>& f)
    {
        cout << "\n---- Source Graph Statistics ----\n";
        auto ops = f->get_ordered_ops();
        cout << "Total nodes: " << ops.size() << endl;
        size_t constant_bytes = 0, parameter_bytes = 0, result_bytes = 0, constants = 0, parameters = 0, results = 0;
        map<string, size_t> op_list;
        set<string> types;
        for (const auto& node : ops)
        {
            for (size_t i = 0; i < node->get_output_size(); ++i)
                types.insert(node->get_output_element_type(i).c_type_string());
            op_list[node->description() + shape_text(node->get_output_shape(0))]++;
            size_t bytes = node->get_output_element_type(0).size() * shape_size(node->get_output_shape(0));
            if (node->is_constant())
                constants++, constant_bytes += bytes;
            else if (node->is_parameter())
                parameters++, parameter_bytes += bytes;
            else if (is_type<op::v0::Result>(node))
                results++, result_bytes += bytes;
        }
        cout << "--\n";
        cout << "Total Constant size: " << constant_bytes << " bytes in " << constants << " constants\n";
        cout << "Total Parameter size: " << parameter_bytes << " bytes in " << parameters << " parameters\n";
        cout << "Total Result size: " << result_bytes << " bytes in " << results << " results\n";
        cout << "--\nTypes used:\n";
        for (const string& t : types)
            cout << "    " << t << "\n";
        cout << "--\n";
        for (const auto& o : op_list)
            cout << o.first << ": " << o.second << " ops" << endl;
    }

    bool path_exists(const string& p)
    {
        struct stat st;
        return ::stat(p.c_str(), &st) == 0;
    }

    void collect_files(const string& dir, vector<string>& out)
    {
        DIR* d = ::opendir(dir.c_str());
        if (!d)
            return;
        while (dirent* e = ::readdir(d))
        {
            string name = e->d_name;
            if (name == "." || name == "..")
                continue;
            string path = dir + "/" + name;
            struct stat st;
            if (::stat(path.c_str(), &st) != 0)
                continue;
            if (S_ISDIR(st.st_mode))
                collect_files(path, out);
            else
                out.push_back(path);
        }
        ::closedir(d);
        sort(out.begin(), out.end());
    }

    const char* kUsage = R"###(
DESCRIPTION
    Benchmark nGraph JSON model with given backend.

SYNOPSIS
        nbench [-f <filename>] [-b <backend>] [-i <iterations>]

OPTIONS
        -f|--file                 Serialized model file
        -b|--backend              Backend to use (e.g. HIP)
        -d|--directory            Directory to scan for models. All models are benchmarked.
        -i|--iterations           Iterations (default: 10)
        -s|--statistics           Display op statistics
        --timing_detail           Gather detailed timing
        -w|--warmup_iterations    Number of warm-up iterations
        --no_copy_data            Disable copy of input/result data every iteration
        --dump_results            Dump result tensors to standard output.
)###";
}

int main(int argc, char** argv)
{
    string model_arg, backend, directory;
    int iterations = 10, warmup_iterations = 1;
    bool failed = false, statistics = false, timing_detail = false, copy_data = true, dump_results = false;

    auto next_int = [&](int& i, int& into) {
        try
        {
            if (i + 1 >= argc)
                throw invalid_argument("missing");
            into = stoi(argv[++i]);
            if (into < 0)
                throw invalid_argument("negative");
        }
        catch (...)
        {
            cout << "Invalid Argument\n";
            failed = true;
        }
    };
    auto next_string = [&](int& i, string& into) {
        if (i + 1 >= argc)
        {
            cout << "Invalid Argument\n";
            failed = true;
            return;
        }
        into = argv[++i];
    };
    for (int i = 1; i < argc; i++)
    {
        string arg = argv[i];
        if (arg == "-f" || arg == "--file")
            next_string(i, model_arg);
        else if (arg == "-b" || arg == "--backend")
            next_string(i, backend);
        else if (arg == "-i" || arg == "--iterations")
            next_int(i, iterations);
        else if (arg == "-s" || arg == "--statistics")
            statistics = true;
        else if (arg == "--timing_detail" || arg == "--timing-detail")
            timing_detail = true;
        else if (arg == "--no_copy_data")
            copy_data = false;
        else if (arg == "--dump_results")
            dump_results = true;
        else if (arg == "-d" || arg == "--directory")
            next_string(i, directory);
        else if (arg == "-w" || arg == "--warmup_iterations")
            next_int(i, warmup_iterations);
        else if (arg == "-v" || arg == "--visualize" || arg == "--dot" || arg == "--double_buffer")
        {
            cout << "Option " << arg << " is not supported by this build\n";
            failed = true;
        }
        else
        {
            cout << "Unknown option: " << arg << endl;
            failed = true;
        }
    }
    if (!model_arg.empty() && !path_exists(model_arg))
    {
        cout << "File " << model_arg << " not found\n";
        failed = true;
    }
    else if (!directory.empty() && !path_exists(directory))
    {
        cout << "Directory " << directory << " not found\n";
        failed = true;
    }
    else if (directory.empty() && model_arg.empty())
    {
        cout << "Either file or directory must be specified\n";
        failed = true;
    }
    if (failed)
    {
        cout << kUsage;
        return 1;
    }

    vector<string> models;
    if (!directory.empty())
        collect_files(directory, models);
    else
        models.push_back(model_arg);

    int rc = 0;
    for (const string& model : models)
    {
        cout << "\n";
        cout << "============================================================================\n";
        cout << "---- Processing '" << model << "'\n";
        cout << "============================================================================\n";
        try
        {
            if (statistics)
                print_statistics(deserialize(model));
            if (!backend.empty())
            {
                cout << "\n---- Benchmark ----\n";
                stopwatch t1;
                t1.start();
                shared_ptr<Function> f = deserialize(model);
                cout << "deserialize took " << t1.elapsed_milliseconds() << "ms\n";
                auto perf_data = run_benchmark(f,
                                               backend,
                                               static_cast<size_t>(iterations),
                                               timing_detail,
                                               static_cast<size_t>(warmup_iterations),
                                               copy_data,
                                               dump_results);
                print_results(perf_data, timing_detail);
            }
        }
        catch (const ngraph::unsupported_op& ue)
        {
            cout << "Unsupported op '" << ue.what() << "' in model " << model << endl;
            rc += 1;
        }
        catch (const exception& e)
        {
            cout << "Exception caught on '" << model << "'\n" << e.what() << endl;
            rc += 1;
        }
    }
    return rc;
}
