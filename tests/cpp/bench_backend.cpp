// hip_backend_tests --bench: the product boundary under a stopwatch.  Each workload is an
// ngraph::Function run as a client of the reference would run it -- Backend::create("HIP"),
// compile, Executable::call -- with the protocol of the reference's nbench
// (src/tools/nbench/benchmark.cpp:141-176) in its --no_copy_data form: inputs written once before the
// loop, warm-up calls, then the timed calls with nothing but Executable::call inside the stopwatch
// (a call returns when the results are in the output tensors).  One JSON object per line on stdout.
#include <chrono>
#include <iostream>
#include <string>

#include "resnet50_graph.hpp"
#include "test_util.hpp"

using namespace std;
using namespace ngraph;

namespace
{
    // BASELINE's first configuration at a batch: op::v0::QuantizedConvolution, u8 NCHW x i8 KCRS -> i8
    shared_ptr<Function> config1_layer(size_t N)
    {
        auto data = make_shared<op::v0::Parameter>(element::u8, Shape{N, 64, 56, 56});
        auto filt = make_shared<op::v0::Constant>(element::i8, Shape{64, 64, 3, 3}, resnet50_graph::uniform_int<int8_t>(1002, 64 * 64 * 9, -127, 127));
        auto f32c = [](float v) { return op::v0::Constant::create(element::f32, Shape{}, {v}); };
        auto u8z = op::v0::Constant::create(element::u8, Shape{}, {0});
        auto i8z = op::v0::Constant::create(element::i8, Shape{}, {0});
        auto conv = make_shared<op::v0::QuantizedConvolution>(data, filt, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1}, Strides{1, 1}, f32c(0.02f), u8z, f32c(0.005f),
                                                              i8z, f32c(0.1f), i8z, element::i8);
        return make_shared<Function>(OutputVector{conv}, ParameterVector{data});
    }

    bool g_detail = false; // --detail: device time of every launch (events around each; nbench's --timing_detail)

    template <typename T>
    void time_function(const string& name, size_t batch, const shared_ptr<Function>& f, const vector<T>& input, size_t warmup, size_t calls, double ops_per_call)
    {
        auto backend = runtime::Backend::create("HIP");
        if (g_detail)
        {
            auto exec = backend->compile(f, true);
            auto in = backend->create_tensor(f->get_parameters().at(0)->get_output_element_type(0), f->get_parameters().at(0)->get_output_shape(0));
            copy_data(in, input);
            auto out = backend->create_tensor(f->get_output_element_type(0), f->get_output_shape(0));
            for (size_t i = 0; i < 5; ++i)
                exec->call({out}, {in});
            double total = 0;
            for (const auto& pc : exec->get_performance_data())
            {
                const auto& n = pc.get_node();
                cout << "  " << n->description() << " -> " << n->get_output_element_type(0).c_type_string() << " [";
                for (size_t d : n->get_output_shape(0))
                    cout << d << " ";
                cout << "] " << static_cast<double>(pc.total_microseconds()) / static_cast<double>(pc.call_count()) << " us" << endl;
                total += static_cast<double>(pc.total_microseconds()) / static_cast<double>(pc.call_count());
            }
            cout << "  " << name << " batch " << batch << ": " << exec->get_performance_data().size() << " launches, " << total << " us of device time a call" << endl;
            return;
        }
        auto exec = backend->compile(f);
        auto param = f->get_parameters().at(0);
        auto in = backend->create_tensor(param->get_output_element_type(0), param->get_output_shape(0));
        copy_data(in, input);
        in->set_stale(false);
        auto out = backend->create_tensor(f->get_output_element_type(0), f->get_output_shape(0));
        for (size_t i = 0; i < warmup; ++i)
            exec->call({out}, {in});
        const auto t0 = chrono::steady_clock::now();
        for (size_t i = 0; i < calls; ++i)
            exec->call({out}, {in});
        const double ms = chrono::duration<double, milli>(chrono::steady_clock::now() - t0).count() / static_cast<double>(calls);
        cout << "{\"workload\": \"" << name << "\", \"batch\": " << batch << ", \"warmup\": " << warmup << ", \"calls\": " << calls << ", \"ms_per_call\": " << ms
             << ", \"per_second\": " << static_cast<double>(batch) / ms * 1e3 << ", \"tops\": " << ops_per_call / (ms * 1e-3) / 1e12 << "}" << endl;
    }
}

int run_backend_bench(int argc, char** argv)
{
    size_t warmup = 10, calls = 100;
    string only;
    for (int i = 1; i < argc; ++i)
    {
        const string a = argv[i];
        if (a == "--calls" && i + 1 < argc)
            calls = static_cast<size_t>(stoul(argv[++i]));
        else if (a == "--warmup" && i + 1 < argc)
            warmup = static_cast<size_t>(stoul(argv[++i]));
        else if (a == "--only" && i + 1 < argc)
            only = argv[++i];
        else if (a == "--detail")
            g_detail = true;
    }
    try
    {
        if (only.empty() || only == "conv")
            time_function("QuantizedConvolution u8[N,64,56,56] x i8[64,64,3,3] -> i8 (BASELINE config 1's layer)", 128, config1_layer(128),
                          resnet50_graph::uniform_int<uint8_t>(1001, size_t(128) * 64 * 56 * 56, 0, 255), warmup, calls, 2.0 * 128 * 64 * 64 * 9 * 56 * 56);
        if (only.empty() || only == "resnet50")
            for (size_t n : {size_t(1), size_t(32), size_t(128)})
            {
                // four distinct images repeated, as the device plan of bench.py is fed
                auto four = resnet50_graph::synthetic_images(n < 4 ? n : 4);
                vector<float> images;
                images.reserve(n * 3 * 224 * 224);
                while (images.size() < n * 3 * 224 * 224)
                    images.insert(images.end(), four.begin(), four.end());
                images.resize(n * 3 * 224 * 224);
                time_function("synthetic int8 ResNet-50 (BASELINE config 4)", n, resnet50_graph::resnet50(n), images, warmup, calls, 2.0 * 4.09e9 * static_cast<double>(n));
            }
    }
    catch (const std::exception& e)
    {
        cerr << "backend bench failed: " << e.what() << endl;
        return 1;
    }
    return 0;
}
