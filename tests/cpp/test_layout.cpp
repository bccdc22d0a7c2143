// The backend's layout assignment (channels-last interiors): a quantized residual block --
// 1x1 convolution, 3x3 convolution, max pool, 1x1 convolution with a residual sum, concat, 1x1
// convolution -- gives byte-identical results with NGRAPH_PASS_ENABLES "HIPLayout:0" (every tensor in
// nGraph's [N, C, H, W]) and with the pass on (only the block's input and output are).  The test
// also reports the time of a call either way.
#include <chrono>
#include <cstdlib>

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

    shared_ptr<Function> residual_block(size_t N, size_t HW)
    {
        Lcg rng{12345u};
        auto x = make_shared<op::v0::Parameter>(element::u8, Shape{N, 64, HW, HW});
        auto scale = [](float v) { return op::v0::Constant::create(element::f32, Shape{}, {v}); };
        auto conv = [&](const Output<Node>& data, size_t K, size_t C, size_t R, bool relu) {
            auto w = random_constant<int8_t>(element::i8, Shape{K, C, R, R}, rng, -20, 20);
            auto b = random_constant<int32_t>(element::i32, Shape{K}, rng, -2000, 2000);
            const ptrdiff_t pad = static_cast<ptrdiff_t>(R / 2);
            return make_shared<op::v0::QuantizedConvolutionBias>(data, w, b, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{pad, pad}, CoordinateDiff{pad, pad}, Strides{1, 1},
                                                                 scale(R == 1 ? 1.0f / 900 : 1.0f / 2500), relu);
        };
        auto c1 = conv(x, 64, 64, 1, true);
        auto c2 = conv(c1, 64, 64, 3, true);
        auto mp = make_shared<op::v0::MaxPool>(c2, Shape{3, 3}, Strides{1, 1}, Shape{1, 1}, Shape{1, 1});
        auto w3 = random_constant<int8_t>(element::i8, Shape{64, 64, 1, 1}, rng, -20, 20);
        auto b3 = random_constant<int32_t>(element::i32, Shape{64}, rng, -2000, 2000);
        auto c3 = make_shared<op::v0::QuantizedConvolutionBiasAdd>(mp, w3, b3, c1, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1}, scale(1.0f / 1100),
                                                                   scale(0.5f), true);
        auto cat = make_shared<op::v0::Concat>(OutputVector{c3, mp}, 1);
        auto c4 = conv(cat, 32, 128, 1, false);
        return make_shared<Function>(OutputVector{c4}, ParameterVector{x});
    }

    vector<int8_t> run_block(size_t N, size_t HW, bool layout_pass, double* us_per_call)
    {
        setenv("NGRAPH_PASS_ENABLES", layout_pass ? "HIPLayout:1" : "HIPLayout:0", 1);
        auto f = residual_block(N, HW);
        auto backend = runtime::Backend::create("HIP");
        auto a = backend->create_tensor(element::u8, f->get_parameters()[0]->get_output_shape(0));
        Lcg rng{777u};
        vector<uint8_t> data(a->get_element_count());
        for (auto& v : data)
            v = static_cast<uint8_t>(rng.next(0, 255));
        copy_data(a, data);
        auto r = backend->create_tensor(element::i8, f->get_output_shape(0));
        auto exec = backend->compile(f);
        unsetenv("NGRAPH_PASS_ENABLES");
        exec->call_with_validate({r}, {a});
        if (us_per_call)
        {
            const int reps = 30;
            auto t0 = chrono::steady_clock::now();
            for (int i = 0; i < reps; ++i)
                exec->call({r}, {a});
            *us_per_call = chrono::duration<double, micro>(chrono::steady_clock::now() - t0).count() / reps;
        }
        return read_vector<int8_t>(r);
    }
}

GPU_TEST(HIP, layout_pass_residual_block)
{
    // 14x14 maps: generic convolution kernels; 56x56 maps at 64 channels: the band kernel
    for (size_t hw : {14u, 56u})
    {
        double us_off = 0, us_on = 0;
        auto off = run_block(4, hw, false, &us_off);
        auto on = run_block(4, hw, true, &us_on);
        EXPECT_TRUE(off == on);
        size_t nonzero = 0;
        for (int8_t v : on)
            nonzero += v != 0;
        EXPECT_TRUE(nonzero > on.size() / 4); // the block computes something
        {
            // device time per op (events around every launch)
            auto f = residual_block(4, hw);
            auto backend = runtime::Backend::create("HIP");
            auto a = backend->create_tensor(element::u8, f->get_parameters()[0]->get_output_shape(0));
            auto r = backend->create_tensor(element::i8, f->get_output_shape(0));
            auto exec = backend->compile(f, true);
            for (int i = 0; i < 10; ++i)
                exec->call({r}, {a});
            for (const auto& pc : exec->get_performance_data())
                std::cout << "[   INFO   ]   " << pc.get_node()->description() << " " << pc.microseconds() << " us" << std::endl;
        }
        std::cout << "[   INFO   ] residual block N=4 " << hw << "x" << hw << ": " << us_off << " us per call in nGraph's layout, " << us_on << " us channels-last inside" << std::endl;
    }
}

// Executable::call replays a HIP graph from its third call with the same tensors on.  Every replay is
// checked against an executable that never captures (NGRAPH_PASS_ENABLES "HIPGraph:0"), with new input
// data before each call and the other executable's eager launches and synchronizations in between.
GPU_TEST(HIP, call_replays_hip_graph)
{
    for (bool layout_pass : {true, false}) // without the layout pass the calls go through the library's workspace
    {
        const size_t N = 2, HW = 56;
        auto backend = runtime::Backend::create("HIP");
        setenv("NGRAPH_PASS_ENABLES", layout_pass ? "HIPGraph:1;HIPLayout:1" : "HIPGraph:1;HIPLayout:0", 1);
        auto with_graph = backend->compile(residual_block(N, HW));
        setenv("NGRAPH_PASS_ENABLES", layout_pass ? "HIPGraph:0;HIPLayout:1" : "HIPGraph:0;HIPLayout:0", 1);
        auto eager = backend->compile(residual_block(N, HW));
        unsetenv("NGRAPH_PASS_ENABLES");
        const Shape in_shape{N, 64, HW, HW}, out_shape{N, 32, HW, HW};
        auto a = backend->create_tensor(element::u8, in_shape);
        auto r1 = backend->create_tensor(element::i8, out_shape);
        auto r2 = backend->create_tensor(element::i8, out_shape);
        auto other = backend->create_tensor(element::i8, out_shape);
        Lcg rng{99u};
        vector<uint8_t> data(shape_size(in_shape));
        for (int call = 0; call < 7; ++call)
        {
            for (auto& v : data)
                v = static_cast<uint8_t>(rng.next(0, 255));
            copy_data(a, data);
            // call 5 writes to another tensor (a new set of addresses: eager again), call 6 returns to the first set
            auto& target = call == 5 ? other : r1;
            with_graph->call_with_validate({target}, {a});
            eager->call_with_validate({r2}, {a});
            EXPECT_TRUE(read_vector<int8_t>(target) == read_vector<int8_t>(r2));
        }
    }
}

// A classifier tail behind residual blocks: QuantizedConvolutionBiasSignedAdd -> Convert (i8 -> u8) ->
// QuantizedConvolutionBiasAdd -> global AvgPool -> Reshape [N, C, 1, 1] -> [N, C] -> QuantizedDotBias.
// Reshape and the GEMM only know nGraph's layout, but a tensor without spatial extent has the same
// bytes either way: the blocks in front stay channels-last (no transposition launches), the Convert
// between the 8-bit types and the transposition-free Reshape are no launches at all, and the
// results equal those of the pass-off run bit for bit.
namespace
{
    shared_ptr<Function> classifier_tail(size_t N)
    {
        Lcg rng{4242u};
        auto x = make_shared<op::v0::Parameter>(element::u8, Shape{N, 64, 7, 7});
        auto scale = [](float v) { return op::v0::Constant::create(element::f32, Shape{}, {v}); };
        auto weights = [&](size_t K, size_t C) { return random_constant<int8_t>(element::i8, Shape{K, C, 1, 1}, rng, -20, 20); };
        auto bias = [&](size_t K) { return random_constant<int32_t>(element::i32, Shape{K}, rng, -2000, 2000); };
        auto c1 = make_shared<op::v0::QuantizedConvolutionBias>(x, weights(64, 64), bias(64), Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1},
                                                                scale(1.0f / 900), true);
        auto down = make_shared<op::v0::QuantizedConvolutionBias>(x, weights(128, 64), bias(128), Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1},
                                                                  scale(1.0f / 1800), false);
        auto c3 = make_shared<op::v0::QuantizedConvolutionBiasSignedAdd>(c1, weights(128, 64), bias(128), down, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0},
                                                                         Strides{1, 1}, scale(1.0f / 1100), scale(0.5f), true);
        auto u = make_shared<op::v0::Convert>(c3, element::u8);
        auto c4 = make_shared<op::v0::QuantizedConvolutionBias>(u, weights(64, 128), bias(64), Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1},
                                                                scale(1.0f / 1300), true);
        auto c5 = make_shared<op::v0::QuantizedConvolutionBiasAdd>(c4, weights(128, 64), bias(128), u, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1},
                                                                   scale(1.0f / 1100), scale(0.5f), true);
        auto pool = make_shared<op::v0::AvgPool>(c5, Shape{7, 7}, Strides{1, 1}, Shape{0, 0}, Shape{0, 0}, false);
        auto flat = make_shared<op::v0::Reshape>(pool, AxisVector{0, 1, 2, 3}, Shape{N, 128});
        auto w = random_constant<int8_t>(element::i8, Shape{48, 128}, rng, -100, 100);
        auto fc = make_shared<op::v0::QuantizedDotBias>(flat, w, bias(48), scale(1.0f / 300), true, false);
        return make_shared<Function>(OutputVector{fc, u}, ParameterVector{x});
    }
}

GPU_TEST(HIP, layout_pass_keeps_blocks_channels_last_in_front_of_a_classifier)
{
    const size_t N = 6;
    vector<int8_t> logits[2];
    vector<uint8_t> block[2];
    size_t launches[2] = {0, 0};
    for (int on = 0; on < 2; ++on)
    {
        setenv("NGRAPH_PASS_ENABLES", on ? "HIPLayout:1" : "HIPLayout:0", 1);
        auto f = classifier_tail(N);
        auto backend = runtime::Backend::create("HIP");
        auto a = backend->create_tensor(element::u8, Shape{N, 64, 7, 7});
        Lcg rng{31u};
        vector<uint8_t> data(a->get_element_count());
        for (auto& v : data)
            v = static_cast<uint8_t>(rng.next(0, 255));
        copy_data(a, data);
        auto r = backend->create_tensor(element::i8, Shape{N, 48});
        auto r2 = backend->create_tensor(element::u8, Shape{N, 128, 7, 7});
        auto exec = backend->compile(f, true);
        unsetenv("NGRAPH_PASS_ENABLES");
        for (int i = 0; i < 3; ++i)
            exec->call_with_validate({r, r2}, {a});
        logits[on] = read_vector<int8_t>(r);
        block[on] = read_vector<uint8_t>(r2);
        launches[on] = exec->get_performance_data().size();
    }
    EXPECT_TRUE(logits[0] == logits[1]);
    EXPECT_TRUE(block[0] == block[1]); // the Convert's value, returned in nGraph's layout either way
    size_t distinct = 0, seen[256] = {0};
    for (int8_t v : logits[1])
        distinct += seen[static_cast<uint8_t>(v)]++ == 0;
    EXPECT_TRUE(distinct > 20);
    // five convolutions, the pool and the GEMM: Convert and Reshape launch nothing
    EXPECT_EQ(launches[0], size_t(7));
    EXPECT_EQ(launches[1], size_t(7));
}

// A network's first two layers: QuantizedConvolutionBias (3 -> 64 channels, 7 x 7, stride 2, ReLU) over
// an NCHW parameter, then MaxPool 3 x 3 / 2.  With the glue fusion on the pair is one launch (the
// convolution's own output is never written); with NGRAPH_PASS_ENABLES "HIPGlueFusion:0" it is two.
// The bytes of the 1 x 1 convolution behind the pool are the same either way.  (The pool itself is not
// returned: a tensor a Result reads is kept in nGraph's layout, and the fused kernel writes channels-last.)
namespace
{
    shared_ptr<Function> first_layers(size_t N, size_t H, size_t W)
    {
        Lcg rng{2024u};
        auto x = make_shared<op::v0::Parameter>(element::u8, Shape{N, 3, H, W});
        auto scale = [](float v) { return op::v0::Constant::create(element::f32, Shape{}, {v}); };
        auto w = random_constant<int8_t>(element::i8, Shape{64, 3, 7, 7}, rng, -100, 100);
        auto b = random_constant<int32_t>(element::i32, Shape{64}, rng, -20000, 20000);
        auto stem = make_shared<op::v0::QuantizedConvolutionBias>(x, w, b, Strides{2, 2}, Strides{1, 1}, CoordinateDiff{3, 3}, CoordinateDiff{3, 3}, Strides{1, 1}, scale(1.0f / 600), true);
        auto pool = make_shared<op::v0::MaxPool>(stem, Shape{3, 3}, Strides{2, 2}, Shape{1, 1}, Shape{1, 1});
        auto w2 = random_constant<int8_t>(element::i8, Shape{32, 64, 1, 1}, rng, -20, 20);
        auto b2 = random_constant<int32_t>(element::i32, Shape{32}, rng, -2000, 2000);
        auto c2 = make_shared<op::v0::QuantizedConvolutionBias>(pool, w2, b2, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1}, scale(1.0f / 100), true);
        return make_shared<Function>(OutputVector{c2}, ParameterVector{x});
    }
}

GPU_TEST(HIP, first_convolution_and_max_pool_are_one_launch)
{
    const size_t N = 3, H = 64, W = 48;
    vector<uint8_t> out[2];
    size_t launches[2] = {0, 0};
    for (int on = 0; on < 2; ++on)
    {
        setenv("NGRAPH_PASS_ENABLES", on ? "HIPGlueFusion:1" : "HIPGlueFusion:0", 1);
        auto f = first_layers(N, H, W);
        auto backend = runtime::Backend::create("HIP");
        auto a = backend->create_tensor(element::u8, Shape{N, 3, H, W});
        Lcg rng{5u};
        vector<uint8_t> data(a->get_element_count());
        for (auto& v : data)
            v = static_cast<uint8_t>(rng.next(0, 255));
        copy_data(a, data);
        auto r = backend->create_tensor(element::u8, f->get_output_shape(0));
        auto exec = backend->compile(f, true);
        unsetenv("NGRAPH_PASS_ENABLES");
        for (int i = 0; i < 3; ++i)
            exec->call_with_validate({r}, {a});
        out[on] = read_vector<uint8_t>(r);
        launches[on] = exec->get_performance_data().size();
    }
    EXPECT_TRUE(out[0] == out[1]);
    size_t distinct = 0, seen[256] = {0};
    for (uint8_t v : out[1])
        distinct += seen[v]++ == 0;
    EXPECT_TRUE(distinct > 50);
    EXPECT_EQ(launches[0], size_t(3)); // convolution, pool, convolution
    EXPECT_EQ(launches[1], size_t(2)); // convolution + pool, convolution
}
