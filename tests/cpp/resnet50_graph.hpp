// The synthetic int8 ResNet-50 of ngraph_amd/resnet50.py as an ngraph::Function (BASELINE's fourth
// configuration: f32 N(0,1) images, Quantize, 53 fused quantized convolutions, two pools, the
// requantizing classifier GEMM, Dequantize), with that module's seeded weights: the generators below
// are its splitmix64 counter generators.  Shared by the backend test and the backend benchmark mode.
#pragma once

#include <cmath>
#include <cstdint>
#include <memory>
#include <vector>

#include "ngraph/ngraph.hpp"

namespace resnet50_graph
{
    using namespace ngraph;
    using std::make_shared;
    using std::shared_ptr;
    using std::vector;

    inline uint64_t splitmix(uint64_t seed, uint64_t i) // word i (from 0) of the stream `seed`
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
    inline vector<float> uniform_f32(uint64_t seed, size_t n, double lo, double hi)
    {
        vector<float> v(n);
        for (size_t i = 0; i < n; ++i)
            v[i] = static_cast<float>(lo + (hi - lo) * (static_cast<double>(splitmix(seed, i) >> 11) * (1.0 / 9007199254740992.0)));
        return v;
    }
    // N(0,1) by Box-Muller over two splitmix64 streams (synth.normal_f32): the first half of the
    // values are r cos, the second half r sin
    inline vector<float> normal_f32(uint64_t seed, size_t n)
    {
        const size_t m = (n + 1) / 2;
        vector<float> v(2 * m);
        for (size_t i = 0; i < m; ++i)
        {
            const double u1 = (static_cast<double>(splitmix(seed, i) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
            const double u2 = static_cast<double>(splitmix(seed, m + i) >> 11) * (1.0 / 9007199254740992.0);
            const double r = std::sqrt(-2.0 * std::log(u1));
            const double phi = (2.0 * 3.141592653589793) * u2;
            v[i] = static_cast<float>(r * std::cos(phi));
            v[m + i] = static_cast<float>(r * std::sin(phi));
        }
        v.resize(n);
        return v;
    }
    // image i of the batch `seed` (resnet50.synthetic_images)
    inline vector<float> synthetic_images(size_t N, uint64_t seed = 42)
    {
        vector<float> all;
        all.reserve(N * 3 * 224 * 224);
        for (size_t i = 0; i < N; ++i)
        {
            const auto one = normal_f32(seed * 1000 + i, 3 * 224 * 224);
            all.insert(all.end(), one.begin(), one.end());
        }
        return all;
    }

    constexpr float kInputScale = 1.0f / 32;
    constexpr int kInputZeroPoint = 128;
    constexpr float kLogitScale = 0.05f;

    struct Net
    {
        int seed = 10;
        // per-channel scales: uniform 0.8 .. 1.2 times the layer's scale, in float
        shared_ptr<Node> scales(int s, size_t K, double scale)
        {
            auto v = uniform_f32(7000 + s, K, 0.8, 1.2);
            const float f = static_cast<float>(scale);
            for (auto& x : v)
                x = x * f;
            return make_shared<op::v0::Constant>(element::f32, Shape{K}, v);
        }
        // a layer hands on the root mean square it was given: sqrt(2) / (rms of the weights x sqrt(reduction))
        static double conv_scale(size_t C, size_t R, double gain) { return gain * std::sqrt(2.0) / (73.3 * std::sqrt(static_cast<double>(C * R * R))); }
        static double stem_scale(size_t C, size_t R) { return 36.0 / ((1.0 / static_cast<double>(kInputScale)) * 73.3 * std::sqrt(static_cast<double>(C * R * R))); }
        shared_ptr<Node> filter(int s, size_t K, size_t C, size_t R) { return make_shared<op::v0::Constant>(element::i8, Shape{K, C, R, R}, uniform_int<int8_t>(1000 + s, K * C * R * R, -127, 127)); }
        shared_ptr<Node> bias(int s, size_t K, int lim) { return make_shared<op::v0::Constant>(element::i32, Shape{K}, uniform_int<int32_t>(5000 + s, K, -lim, lim)); }

        shared_ptr<Node> conv(const Output<Node>& x, int s, size_t C, size_t K, size_t R, size_t stride, bool relu, double gain = 1.0)
        {
            const ptrdiff_t pad = static_cast<ptrdiff_t>(R / 2);
            return make_shared<op::v0::QuantizedConvolutionBias>(x, filter(s, K, C, R), bias(s, K, 3000), Strides{stride, stride}, Strides{1, 1}, CoordinateDiff{pad, pad}, CoordinateDiff{pad, pad},
                                                                 Strides{1, 1}, scales(s, K, conv_scale(C, R, gain)), relu);
        }
        // the stem: the input's zero point folded into the bias, sum((x - zp) w) = sum(x w) - zp sum(w)
        shared_ptr<Node> stem(const Output<Node>& x)
        {
            const size_t K = 64, C = 3, R = 7;
            const auto w = uniform_int<int8_t>(1000 + 1, K * C * R * R, -127, 127);
            auto b = uniform_int<int32_t>(5000 + 1, K, -3000, 3000);
            for (size_t k = 0; k < K; ++k)
            {
                int32_t sum = 0;
                for (size_t i = 0; i < C * R * R; ++i)
                    sum += w[k * C * R * R + i];
                b[k] -= kInputZeroPoint * sum;
            }
            return make_shared<op::v0::QuantizedConvolutionBias>(x, make_shared<op::v0::Constant>(element::i8, Shape{K, C, R, R}, w), make_shared<op::v0::Constant>(element::i32, Shape{K}, b),
                                                                 Strides{2, 2}, Strides{1, 1}, CoordinateDiff{3, 3}, CoordinateDiff{3, 3}, Strides{1, 1}, scales(1, K, stem_scale(C, R)), true);
        }
    };

    inline shared_ptr<Function> resnet50(size_t N)
    {
        Net net;
        auto image = make_shared<op::v0::Parameter>(element::f32, Shape{N, 3, 224, 224});
        auto in_scale = op::v0::Constant::create(element::f32, Shape{}, {kInputScale});
        auto in_zp = op::v0::Constant::create(element::u8, Shape{}, {kInputZeroPoint});
        auto image8 = make_shared<op::v0::Quantize>(image, in_scale, in_zp, element::u8, AxisSet{}, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
        shared_ptr<Node> x = net.stem(image8);
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
                                                                                     net.scales(sd + 3, cout, Net::conv_scale(mid, 1, 0.85)), half, true);
                    x = make_shared<op::v0::Convert>(c3, element::u8);
                }
                else
                    x = make_shared<op::v0::QuantizedConvolutionBiasAdd>(c2, net.filter(sd + 3, cout, mid, 1), net.bias(sd + 3, cout, 3000), x, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0},
                                                                         CoordinateDiff{0, 0}, Strides{1, 1}, net.scales(sd + 3, cout, Net::conv_scale(mid, 1, 0.85)), half, true);
                cin = cout;
                net.seed += 4;
            }
        }
        x = make_shared<op::v0::AvgPool>(x, Shape{7, 7}, Strides{1, 1}, Shape{0, 0}, Shape{0, 0}, false);
        x = make_shared<op::v0::Reshape>(x, AxisVector{0, 1, 2, 3}, Shape{N, 2048});
        const int sd = net.seed;
        auto w = make_shared<op::v0::Constant>(element::i8, Shape{1000, 2048}, uniform_int<int8_t>(1000 + sd, 1000 * 2048, -127, 127));
        auto fc = make_shared<op::v0::QuantizedDotBias>(x, w, net.bias(sd, 1000, 20000), net.scales(sd, 1000, 1.0 / 400), true, false);
        auto out_scale = op::v0::Constant::create(element::f32, Shape{}, {kLogitScale});
        auto out_zp = op::v0::Constant::create(element::i8, Shape{}, {0});
        auto logits = make_shared<op::v0::Dequantize>(fc, out_scale, out_zp, element::f32, AxisSet{});
        return make_shared<Function>(OutputVector{logits}, ParameterVector{image});
    }
}
