// The synthetic int8 ResNet-50 as an ngraph::Function on backend "HIP": the same network as
// ngraph_amd/resnet50.py (same seeded weights: the generator below is that module's splitmix64
// counter generator), built from QuantizedConvolutionBias / BiasAdd / BiasSignedAdd, MaxPool, AvgPool,
// Convert, Reshape and QuantizedDotBias nodes, compiled and called like any other function.  Its
// logits for the seeded image must equal, bit for bit, the ones the CPU restatement of the ops
// computes (tests/golden/resnet50_logits.npz, tabled in resnet50_logits.inc).
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <cstring>

#include "test_util.hpp"

using namespace std;
using namespace ngraph;

#include "resnet50_logits.inc"

namespace
{
    uint64_t splitmix(uint64_t seed, uint64_t i) // word i (from 0) of the stream `seed`
    {
        uint64_t z = (i + 1) * 0x9E3779B97F4A7C15ull + seed;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    template <typename T>
    vector<T> uniform_int(uint64_t seed, size_t n, int lo, int hi)
    {
        vector<T> v(n);
        const uint64_t span = static_cast<uint64_t>(hi - lo + 1);
        for (size_t i = 0; i < n; ++i)
            v[i] = static_cast<T>(static_cast<int64_t>((splitmix(seed, i) >> 11) % span) + lo);
        return v;
    }
    vector<float> uniform_f32(uint64_t seed, size_t n, double lo, double hi)
    {
        vector<float> v(n);
        for (size_t i = 0; i < n; ++i)
            v[i] = static_cast<float>(lo + (hi - lo) * (static_cast<double>(splitmix(seed, i) >> 11) * (1.0 / 9007199254740992.0)));
        return v;
    }

    struct Net
    {
        int seed = 10;
        // per-channel scales: uniform 0.8 .. 1.2 times gain * 48 / (73 * 80 * sqrt(C * R * R)), in float
        shared_ptr<Node> scales(int s, size_t K, double scale)
        {
            auto v = uniform_f32(7000 + s, K, 0.8, 1.2);
            const float f = static_cast<float>(scale);
            for (auto& x : v)
                x = x * f;
            return make_shared<op::v0::Constant>(element::f32, Shape{K}, v);
        }
        static double conv_scale(size_t C, size_t R, double gain) { return gain * 48.0 / (73.0 * 80.0 * sqrt(static_cast<double>(C * R * R))); }
        shared_ptr<Node> filter(int s, size_t K, size_t C, size_t R) { return make_shared<op::v0::Constant>(element::i8, Shape{K, C, R, R}, uniform_int<int8_t>(1000 + s, K * C * R * R, -127, 127)); }
        shared_ptr<Node> bias(int s, size_t K, int lim) { return make_shared<op::v0::Constant>(element::i32, Shape{K}, uniform_int<int32_t>(5000 + s, K, -lim, lim)); }

        shared_ptr<Node> conv(const Output<Node>& x, int s, size_t C, size_t K, size_t R, size_t stride, bool relu, double gain = 1.0)
        {
            const ptrdiff_t pad = static_cast<ptrdiff_t>(R / 2);
            return make_shared<op::v0::QuantizedConvolutionBias>(x, filter(s, K, C, R), bias(s, K, 3000), Strides{stride, stride}, Strides{1, 1}, CoordinateDiff{pad, pad}, CoordinateDiff{pad, pad},
                                                                 Strides{1, 1}, scales(s, K, conv_scale(C, R, gain)), relu);
        }
    };

    shared_ptr<Function> resnet50(size_t N)
    {
        Net net;
        auto image = make_shared<op::v0::Parameter>(element::u8, Shape{N, 3, 224, 224});
        shared_ptr<Node> x = net.conv(image, 1, 3, 64, 7, 2, true, 0.6);
        x = make_shared<op::v0::MaxPool>(x, Shape{3, 3}, Strides{2, 2}, Shape{1, 1}, Shape{1, 1});
        const size_t stages[4][4] = {{64, 256, 3, 1}, {128, 512, 4, 2}, {256, 1024, 6, 2}, {512, 2048, 3, 2}};
        size_t cin = 64;
        auto half = op::v0::Constant::create(element::f32, Shape{}, {0.5f});
        for (const auto& st : stages)
        {
            const size_t mid = st[0], cout = st[1];
            for (size_t b = 0; b < st[2]; ++b)
            {
                const size_t s = b == 0 ? st[3] : 1;
                const int sd = net.seed;
                auto c1 = net.conv(x, sd, cin, mid, 1, 1, true);
                auto c2 = net.conv(c1, sd + 1, mid, mid, 3, s, true);
                if (b == 0)
                {
                    auto down = net.conv(x, sd + 2, cin, cout, 1, s, false, 0.5);
                    auto c3 = make_shared<op::v0::QuantizedConvolutionBiasSignedAdd>(c2, net.filter(sd + 3, cout, mid, 1), net.bias(sd + 3, cout, 3000), down, Strides{1, 1}, Strides{1, 1},
                                                                                     CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1},
                                                                                     net.scales(sd + 3, cout, Net::conv_scale(mid, 1, 0.7)), half, true);
                    x = make_shared<op::v0::Convert>(c3, element::u8);
                }
                else
                    x = make_shared<op::v0::QuantizedConvolutionBiasAdd>(c2, net.filter(sd + 3, cout, mid, 1), net.bias(sd + 3, cout, 3000), x, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0},
                                                                         CoordinateDiff{0, 0}, Strides{1, 1}, net.scales(sd + 3, cout, Net::conv_scale(mid, 1, 0.7)), half, true);
                cin = cout;
                net.seed += 4;
            }
        }
        x = make_shared<op::v0::AvgPool>(x, Shape{7, 7}, Strides{1, 1}, Shape{0, 0}, Shape{0, 0}, false);
        x = make_shared<op::v0::Reshape>(x, AxisVector{0, 1, 2, 3}, Shape{N, 2048});
        const int sd = net.seed;
        auto w = make_shared<op::v0::Constant>(element::i8, Shape{1000, 2048}, uniform_int<int8_t>(1000 + sd, 1000 * 2048, -127, 127));
        auto logits = make_shared<op::v0::QuantizedDotBias>(x, w, net.bias(sd, 1000, 20000), net.scales(sd, 1000, 1.0 / 4000), false, false);
        return make_shared<Function>(OutputVector{logits}, ParameterVector{image});
    }
}

CPU_TEST(resnet50, graph_shape)
{
    auto f = resnet50(2);
    EXPECT_EQ(f->get_output_shape(0), (Shape{2, 1000}));
    EXPECT_EQ(f->get_output_element_type(0), element::f32);
    EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolutionBias>(f), 37u); // stem + 16 x 2 + 4 shortcuts
    EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolutionBiasAdd>(f), 12u);
    EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolutionBiasSignedAdd>(f), 4u);
}

GPU_TEST(HIP, resnet50_function_matches_reference_logits)
{
    auto backend = runtime::Backend::create("HIP");
    auto image = backend->create_tensor(element::u8, Shape{1, 3, 224, 224});
    copy_data(image, uniform_int<uint8_t>(42, 3 * 224 * 224, 0, 255));
    auto logits = backend->create_tensor(element::f32, Shape{1, 1000});
    auto exec = backend->compile(resnet50(1));
    for (int call = 0; call < 4; ++call) // eager, captured, replayed twice
    {
        exec->call_with_validate({logits}, {image});
        auto got = read_vector<float>(logits);
        size_t same = 0;
        for (size_t i = 0; i < 1000; ++i)
        {
            uint32_t bits;
            memcpy(&bits, &got[i], 4);
            same += bits == kResnet50LogitBits[i];
        }
        EXPECT_EQ(same, 1000u);
    }
    // images per second through Executable::call, batch 32 (the call synchronizes)
    const size_t N = 32;
    auto batch = backend->create_tensor(element::u8, Shape{N, 3, 224, 224});
    copy_data(batch, uniform_int<uint8_t>(43, N * 3 * 224 * 224, 0, 255));
    auto out = backend->create_tensor(element::f32, Shape{N, 1000});
    auto exec32 = backend->compile(resnet50(N));
    for (int i = 0; i < 3; ++i)
        exec32->call({out}, {batch});
    const int reps = 10;
    auto t0 = chrono::steady_clock::now();
    for (int i = 0; i < reps; ++i)
        exec32->call({out}, {batch});
    const double ms = chrono::duration<double, milli>(chrono::steady_clock::now() - t0).count() / reps;
    std::cout << "[   INFO   ] ResNet-50 through Executable::call, batch " << N << ": " << ms << " ms per call, " << N / ms * 1e3 << " images/s" << std::endl;
}
