// Two executables of one backend called from two host threads at once.  The reference allows
// concurrent calls (src/ngraph/runtime/cpu/cpu_call_frame.cpp:119-140); here every executable has a
// stream of its own and the library's scratch blocks (transposed input, partial sums and tile
// counters of reductions split over workgroups) belong to the stream that uses them, so the two
// calls share nothing.  The graphs are deep layers at a small batch -- few output tiles, long
// reductions, which is where reductions get split -- fed in nGraph's [N, C, H, W] layout, which
// goes through the transposition scratch.  Results must equal the same executables' serial results.
#include <atomic>
#include <thread>

#include "test_util.hpp"

using namespace std;
using namespace ngraph;

namespace
{
    struct Lcg
    {
        uint32_t s;
        int next(int lo, int hi)
        {
            s = s * 1664525u + 1013904223u;
            return lo + static_cast<int>((s >> 8) % static_cast<uint32_t>(hi - lo + 1));
        }
    };

    template <typename T>
    shared_ptr<Node> random_constant(const element::Type& et, const Shape& shape, Lcg& rng, int lo, int hi)
    {
        vector<T> v(shape_size(shape));
        for (auto& x : v)
            x = static_cast<T>(rng.next(lo, hi));
        return make_shared<op::v0::Constant>(et, shape, v);
    }

    shared_ptr<Function> deep_layers(size_t N, uint32_t seed)
    {
        Lcg rng{seed};
        auto x = make_shared<op::v0::Parameter>(element::u8, Shape{N, 256, 7, 7});
        auto conv = [&](const Output<Node>& data, size_t K, size_t C, size_t R, bool relu, float s) {
            auto w = random_constant<int8_t>(element::i8, Shape{K, C, R, R}, rng, -20, 20);
            auto b = random_constant<int32_t>(element::i32, Shape{K}, rng, -2000, 2000);
            const ptrdiff_t pad = static_cast<ptrdiff_t>(R / 2);
            return make_shared<op::v0::QuantizedConvolutionBias>(data, w, b, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{pad, pad}, CoordinateDiff{pad, pad}, Strides{1, 1},
                                                                 op::v0::Constant::create(element::f32, Shape{}, {s}), relu);
        };
        auto c1 = conv(x, 256, 256, 3, true, 1.0f / 2500);
        auto c2 = conv(c1, 512, 256, 3, true, 1.0f / 500);
        auto c3 = conv(c2, 64, 512, 1, false, 1.0f / 200);
        return make_shared<Function>(OutputVector{c3}, ParameterVector{x});
    }
}

GPU_TEST(HIP, concurrent_calls_of_two_executables)
{
    const size_t N = 2;
    const int calls = 12;
    auto backend = runtime::Backend::create("HIP");
    shared_ptr<runtime::Executable> exec[2] = {backend->compile(deep_layers(N, 1u)), backend->compile(deep_layers(N, 2u))};
    const Shape in_shape{N, 256, 7, 7}, out_shape{N, 64, 7, 7};
    // inputs of every call, and the serial results
    vector<vector<uint8_t>> inputs[2];
    vector<vector<int8_t>> serial[2];
    for (int e = 0; e < 2; ++e)
    {
        Lcg rng{100u + e};
        auto a = backend->create_tensor(element::u8, in_shape);
        auto r = backend->create_tensor(element::i8, out_shape);
        for (int c = 0; c < calls; ++c)
        {
            vector<uint8_t> data(shape_size(in_shape));
            for (auto& v : data)
                v = static_cast<uint8_t>(rng.next(0, 255));
            copy_data(a, data);
            exec[e]->call_with_validate({r}, {a});
            inputs[e].push_back(data);
            serial[e].push_back(read_vector<int8_t>(r));
        }
        size_t nonzero = 0;
        for (int8_t v : serial[e].back())
            nonzero += v != 0;
        EXPECT_TRUE(nonzero > serial[e].back().size() / 4);
    }
    EXPECT_FALSE(serial[0].back() == serial[1].back()); // two different networks
    // the same calls from two threads at once (new tensors: eager, captured, then replayed calls)
    atomic<int> mismatches{0}, errors{0};
    auto worker = [&](int e) {
        try
        {
            auto a = backend->create_tensor(element::u8, in_shape);
            auto r = backend->create_tensor(element::i8, out_shape);
            for (int round = 0; round < 3; ++round)
                for (int c = 0; c < calls; ++c)
                {
                    copy_data(a, inputs[e][c]);
                    exec[e]->call({r}, {a});
                    if (read_vector<int8_t>(r) != serial[e][c])
                        ++mismatches;
                }
        }
        catch (const std::exception& ex)
        {
            std::cout << "worker " << e << " threw: " << ex.what() << std::endl;
            ++errors;
        }
    };
    thread t0(worker, 0), t1(worker, 1);
    t0.join();
    t1.join();
    EXPECT_EQ(errors.load(), 0);
    EXPECT_EQ(mismatches.load(), 0);
}
