// HIPQuantFusion, after the reference's tests of CPUQuantFusion (test/cpu_fusion.in.cpp:2475-3020):
// the same graphs, run through the backend with the pass switched off and on by
// NGRAPH_PASS_ENABLES and compared, plus the structure the pass leaves (run directly on the
// function: the backend rewrites a private copy, not the caller's graph).  Inputs are multiples of
// the quantization scales, so every requantization is exact and the two rounding policies (the
// plain ops' round-half-away, the fused ops' round-half-even) cannot differ.
#include <cstdlib>

#include "ngraph/runtime/hip/pass/hip_quant_fusion.hpp"
#include "test_util.hpp"

using namespace std;
using namespace ngraph;

namespace
{
    const auto RNE = op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN;

    shared_ptr<Node> f32c(float v) { return op::v0::Constant::create(element::f32, Shape{}, {v}); }
    shared_ptr<Node> i8zero() { return op::v0::Constant::create(element::i8, Shape{}, {0}); }
    shared_ptr<Node> u8zero() { return op::v0::Constant::create(element::u8, Shape{}, {0}); }
    shared_ptr<Node> i32zero() { return op::v0::Constant::create(element::i32, Shape{}, {0}); }

    void run_pass(const shared_ptr<Function>& f)
    {
        runtime::hip::pass::HIPQuantFusion p;
        p.run_on_function(f);
    }

    // f32 parameters in, f32 results out, pass on or off
    vector<vector<float>> execute(const shared_ptr<Function>& f, const vector<vector<float>>& args, bool fuse)
    {
        setenv("NGRAPH_PASS_ENABLES", fuse ? "HIPQuantFusion:1" : "HIPQuantFusion:0", 1);
        auto backend = runtime::Backend::create("HIP");
        vector<shared_ptr<runtime::Tensor>> in, out;
        for (size_t i = 0; i < args.size(); ++i)
        {
            auto t = backend->create_tensor(element::f32, f->get_parameters()[i]->get_output_shape(0));
            copy_data(t, args[i]);
            in.push_back(t);
        }
        for (size_t i = 0; i < f->get_output_size(); ++i)
            out.push_back(backend->create_tensor(f->get_output_element_type(i), f->get_output_shape(i)));
        backend->compile(f)->call_with_validate(out, in);
        unsetenv("NGRAPH_PASS_ENABLES");
        vector<vector<float>> r;
        for (auto& t : out)
            r.push_back(read_vector<float>(t));
        return r;
    }

    // values k * step for k cycling through lo .. hi
    vector<float> ramp(size_t n, float step, int lo, int hi)
    {
        vector<float> v(n);
        for (size_t i = 0; i < n; ++i)
            v[i] = step * static_cast<float>(lo + static_cast<int>((i * 5 + i / 3) % static_cast<size_t>(hi - lo + 1)));
        return v;
    }

    shared_ptr<Function> make_qconv_relu(bool with_bias)
    {
        Shape shape_input{1, 2, 4, 4}, shape_weights{3, 2, 1, 1};
        auto input = make_shared<op::v0::Parameter>(element::f32, shape_input);
        auto weights = make_shared<op::v0::Parameter>(element::f32, shape_weights);
        auto bias = make_shared<op::v0::Parameter>(element::f32, Shape{3});
        auto input_scale = f32c(2.0f), weights_scale = f32c(2.0f), output_scale = f32c(4.0f);
        auto q_input = make_shared<op::v0::Quantize>(input, input_scale, u8zero(), element::u8, AxisSet{}, RNE);
        auto q_weights = make_shared<op::v0::Quantize>(weights, weights_scale, i8zero(), element::i8, AxisSet{}, RNE);
        shared_ptr<Node> conv;
        ParameterVector params{input, weights};
        if (with_bias)
        {
            auto q_bias = make_shared<op::v0::Quantize>(bias, input_scale * weights_scale, i32zero(), element::i32, AxisSet{}, RNE);
            auto requant = (input_scale * weights_scale) / output_scale;
            conv = make_shared<op::v0::QuantizedConvolutionBias>(q_input, q_weights, q_bias, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1}, requant);
            params.push_back(bias);
        }
        else
            conv = make_shared<op::v0::QuantizedConvolution>(q_input, q_weights, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1}, input_scale,
                                                             u8zero(), weights_scale, i8zero(), output_scale, i8zero(), element::i8, AxisSet{}, AxisSet{}, AxisSet{});
        auto dq = make_shared<op::v0::Dequantize>(conv, output_scale, i8zero(), element::f32, AxisSet{});
        auto relu = make_shared<op::v0::Relu>(dq);
        auto q = make_shared<op::v0::Quantize>(relu, output_scale, u8zero(), element::u8, AxisSet{}, RNE);
        auto q_f = make_shared<op::v0::Dequantize>(q, output_scale, u8zero(), element::f32, AxisSet{});
        return make_shared<Function>(OutputVector{q_f}, params);
    }

    shared_ptr<Function> make_qpool(bool avg)
    {
        auto input = make_shared<op::v0::Parameter>(element::f32, Shape{1, 2, 4, 4});
        auto scale = f32c(2.0f);
        auto q_input = make_shared<op::v0::Quantize>(input, scale, u8zero(), element::u8, AxisSet{}, RNE);
        auto dq = make_shared<op::v0::Dequantize>(q_input, scale, u8zero(), element::f32, AxisSet{});
        shared_ptr<Node> pool;
        if (avg)
            pool = make_shared<op::v0::AvgPool>(dq, Shape{2, 2}, Strides{2, 2}, Shape{0, 0}, Shape{0, 0}, false);
        else
            pool = make_shared<op::v0::MaxPool>(dq, Shape{2, 2}, Strides{1, 1}, Shape{0, 0}, Shape{0, 0});
        return make_shared<Function>(OutputVector{pool}, ParameterVector{input});
    }

    shared_ptr<Function> make_qconcat(size_t n_inputs, bool same_scales)
    {
        OutputVector pieces;
        ParameterVector inputs;
        for (size_t i = 0; i < n_inputs; ++i)
        {
            inputs.push_back(make_shared<op::v0::Parameter>(element::f32, Shape{1, 2, 4, 4}));
            auto scale = f32c(same_scales || i == 0 ? 2.0f : 4.0f);
            auto q = make_shared<op::v0::Quantize>(inputs.back(), scale, u8zero(), element::u8, AxisSet{}, RNE);
            pieces.push_back(make_shared<op::v0::Dequantize>(q, scale, u8zero(), element::f32, AxisSet{}));
        }
        return make_shared<Function>(OutputVector{make_shared<op::v0::Concat>(pieces, 1)}, inputs);
    }

    shared_ptr<Function> make_dq_q(bool match_scales, bool match_et)
    {
        auto input = make_shared<op::v0::Parameter>(element::i8, Shape{1, 2, 2});
        auto dq = make_shared<op::v0::Dequantize>(input, f32c(2.0f), i8zero(), element::f32, AxisSet{});
        auto q_scale = f32c(match_scales ? 2.0f : 1.0f);
        shared_ptr<Node> q;
        if (match_et)
            q = make_shared<op::v0::Quantize>(dq, q_scale, i8zero(), element::i8, AxisSet{}, RNE);
        else
            q = make_shared<op::v0::Quantize>(dq, q_scale, u8zero(), element::u8, AxisSet{}, RNE);
        return make_shared<Function>(OutputVector{q}, ParameterVector{input});
    }

    // Relu(Dequantize(QuantizedConvolutionBias) + Dequantize(summand)); the summand is i8 (signed add)
    // or u8, and comes out of a Quantize (a Parameter must not be overwritten in place)
    shared_ptr<Function> make_qconvb_add(bool signed_summand, bool through_reshape)
    {
        Shape shape_input{1, 2, 2, 2}, shape_weights{1, 2, 1, 1}, shape_summand{1, 1, 2, 2};
        auto input = make_shared<op::v0::Parameter>(element::f32, shape_input);
        auto weights = make_shared<op::v0::Parameter>(element::f32, shape_weights);
        auto bias = make_shared<op::v0::Parameter>(element::f32, Shape{1});
        auto summand = make_shared<op::v0::Parameter>(element::f32, shape_summand);
        auto input_scale = f32c(2.0f), weights_scale = f32c(2.0f), output_scale = f32c(4.0f), summand_scale = f32c(2.0f);
        auto q_input = make_shared<op::v0::Quantize>(input, input_scale, u8zero(), element::u8, AxisSet{}, RNE);
        auto q_weights = make_shared<op::v0::Quantize>(weights, weights_scale, i8zero(), element::i8, AxisSet{}, RNE);
        auto q_bias = make_shared<op::v0::Quantize>(bias, input_scale * weights_scale, i32zero(), element::i32, AxisSet{}, RNE);
        shared_ptr<Node> q_summand;
        if (signed_summand)
            q_summand = make_shared<op::v0::Quantize>(summand, summand_scale, i8zero(), element::i8, AxisSet{}, RNE);
        else
            q_summand = make_shared<op::v0::Quantize>(summand, summand_scale, u8zero(), element::u8, AxisSet{}, RNE);
        auto requant = (input_scale * weights_scale) / output_scale;
        auto conv = make_shared<op::v0::QuantizedConvolutionBias>(q_input, q_weights, q_bias, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1}, requant);
        shared_ptr<Node> left = make_shared<op::v0::Dequantize>(conv, output_scale, i8zero(), element::f32, AxisSet{});
        shared_ptr<Node> right = make_shared<op::v0::Dequantize>(q_summand, summand_scale, signed_summand ? i8zero() : u8zero(), element::f32, AxisSet{});
        if (through_reshape)
        {
            left = make_shared<op::v0::Broadcast>(make_shared<op::v0::Reshape>(left, AxisVector{0, 1, 2, 3}, Shape{1, 2, 2}), Shape{1, 1, 2, 2}, AxisSet{0});
            right = make_shared<op::v0::Broadcast>(make_shared<op::v0::Reshape>(right, AxisVector{0, 1, 2, 3}, Shape{1, 2, 2}), Shape{1, 1, 2, 2}, AxisSet{0});
        }
        auto relu = make_shared<op::v0::Relu>(left + right);
        return make_shared<Function>(OutputVector{relu}, ParameterVector{input, weights, bias, summand});
    }
}

// ---- structure ---------------------------------------------------------------------------------

CPU_TEST(hip_quant_fusion, qconv_relu_structure)
{
    auto f = make_qconv_relu(false);
    run_pass(f);
    EXPECT_EQ(count_ops_of_type<op::v0::Relu>(f), 0u);
    EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolution>(f), 0u);
    EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolutionRelu>(f), 1u);
    // Dequantize(conv) -> Quantize -> Dequantize collapses too: same scale, zero points 0, u8 on both sides
    EXPECT_EQ(count_ops_of_type<op::v0::Dequantize>(f), 1u);
    auto g = make_qconv_relu(true);
    run_pass(g);
    EXPECT_EQ(count_ops_of_type<op::v0::Relu>(g), 0u);
    EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolutionBias>(g), 1u);
    for (const auto& n : g->get_ordered_ops())
        if (auto c = as_type_ptr<op::v0::QuantizedConvolutionBias>(n))
        {
            EXPECT_TRUE(c->with_relu());
            EXPECT_EQ(c->get_output_element_type(0), element::u8);
        }
}

CPU_TEST(hip_quant_fusion, pool_and_concat_structure)
{
    for (bool avg : {false, true})
    {
        auto f = make_qpool(avg);
        run_pass(f);
        // the pool now reads the u8 tensor and the Dequantize is the function's result
        EXPECT_TRUE(is_type<op::v0::Dequantize>(f->get_output_op(0)->get_argument(0)));
        for (const auto& n : f->get_ordered_ops())
            if (is_type<op::v0::MaxPool>(n) || is_type<op::v0::AvgPool>(n))
                EXPECT_EQ(n->get_input_element_type(0), element::u8);
    }
    auto f = make_qconcat(7, true);
    run_pass(f);
    EXPECT_EQ(count_ops_of_type<op::v0::Dequantize>(f), 1u);
    for (const auto& n : f->get_ordered_ops())
        if (is_type<op::v0::Concat>(n))
            EXPECT_EQ(n->get_output_element_type(0), element::u8);
    auto g = make_qconcat(3, false); // scales differ: stays a float concat
    run_pass(g);
    EXPECT_EQ(count_ops_of_type<op::v0::Dequantize>(g), 3u);
}

CPU_TEST(hip_quant_fusion, dq_q_structure)
{
    auto fuse = make_dq_q(true, true), no_fuse1 = make_dq_q(false, true), no_fuse2 = make_dq_q(true, false);
    run_pass(fuse);
    run_pass(no_fuse1);
    run_pass(no_fuse2);
    EXPECT_EQ(count_ops_of_type<op::v0::Quantize>(fuse), 0u);
    EXPECT_EQ(count_ops_of_type<op::v0::Quantize>(no_fuse1), 1u);
    EXPECT_EQ(count_ops_of_type<op::v0::Quantize>(no_fuse2), 1u);
}

CPU_TEST(hip_quant_fusion, qconvb_add_structure)
{
    for (bool through_reshape : {false, true})
    {
        auto f = make_qconvb_add(true, through_reshape);
        run_pass(f);
        EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolutionBiasSignedAdd>(f), 1u);
        EXPECT_EQ(count_ops_of_type<op::v0::Convert>(f), 1u);
        EXPECT_EQ(count_ops_of_type<op::v1::Add>(f), 0u);
        EXPECT_EQ(count_ops_of_type<op::v0::Relu>(f), 0u);
        auto g = make_qconvb_add(false, through_reshape);
        run_pass(g);
        EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolutionBiasAdd>(g), 1u);
        EXPECT_EQ(count_ops_of_type<op::v1::Add>(g), 0u);
    }
}

CPU_TEST(hip_quant_fusion, pass_config_switch)
{
    // NGRAPH_PASS_ENABLES is parsed by PassConfig (src/ngraph/pass/pass_config.cpp:27-84); a Manager runs
    // whatever is registered, and it is the registering backend that leaves a pass out when its knob says
    // 0 (src/ngraph/runtime/cpu/cpu_external_function.cpp:215-226) -- the HIP backend's side of it is in
    // the pass-off / pass-on tests below
    setenv("NGRAPH_PASS_ENABLES", "HIPQuantFusion:0;Other:1;Bare", 1);
    pass::PassConfig config;
    EXPECT_EQ(config.get_enables().size(), 3u);
    EXPECT_FALSE(config.get_enables().at("HIPQuantFusion"));
    EXPECT_TRUE(config.get_enables().at("Other"));
    EXPECT_TRUE(config.get_enables().at("Bare"));
    EXPECT_FALSE(config.get_pass_enable("HIPQuantFusion"));
    EXPECT_FALSE(config.get_pass_enable("NotNamed"));
    auto f = make_dq_q(true, true);
    pass::Manager pm; // the knob does not reach a Manager: the registered pass runs
    pm.register_pass<runtime::hip::pass::HIPQuantFusion>();
    pm.run_passes(f);
    EXPECT_EQ(count_ops_of_type<op::v0::Quantize>(f), 0u);
    unsetenv("NGRAPH_PASS_ENABLES");
}

// ---- results, pass off against pass on ------------------------------------------------------------

GPU_TEST(HIP, quant_fusion_qconv_relu)
{
    for (bool with_bias : {false, true})
    {
        vector<vector<float>> args{ramp(32, 2.0f, 0, 9), ramp(6, 2.0f, -3, 3)};
        if (with_bias)
            args.push_back(ramp(3, 4.0f, -5, 5));
        auto off = execute(make_qconv_relu(with_bias), args, false);
        auto on = execute(make_qconv_relu(with_bias), args, true);
        EXPECT_VEC_EQ(off.at(0), on.at(0));
        bool some_positive = false, some_clipped = false;
        for (float v : on.at(0))
        {
            some_positive |= v > 0;
            some_clipped |= v == 0;
        }
        EXPECT_TRUE(some_positive && some_clipped); // the Relu did something on both sides
    }
}

GPU_TEST(HIP, quant_fusion_pools_and_concat)
{
    for (bool avg : {false, true})
    {
        // multiples of 8: the average of four quantized values is then a whole number, so averaging
        // the u8 codes (pass on) and averaging the dequantized floats (pass off) agree exactly
        vector<vector<float>> args{ramp(32, 8.0f, 0, 15)};
        EXPECT_VEC_EQ(execute(make_qpool(avg), args, false).at(0), execute(make_qpool(avg), args, true).at(0));
    }
    vector<vector<float>> args;
    for (int i = 0; i < 7; ++i)
        args.push_back(ramp(32, 2.0f, i, 20 + i));
    EXPECT_VEC_EQ(execute(make_qconcat(7, true), args, false).at(0), execute(make_qconcat(7, true), args, true).at(0));
}

GPU_TEST(HIP, quant_fusion_dq_q)
{
    for (bool fuse : {false, true})
    {
        setenv("NGRAPH_PASS_ENABLES", fuse ? "HIPQuantFusion:1" : "HIPQuantFusion:0", 1);
        auto f = make_dq_q(true, true);
        auto backend = runtime::Backend::create("HIP");
        auto a = backend->create_tensor(element::i8, Shape{1, 2, 2});
        copy_data(a, vector<int8_t>{-1, 2, 3, 4});
        auto r = backend->create_tensor(element::i8, Shape{1, 2, 2});
        backend->compile(f)->call_with_validate({r}, {a});
        EXPECT_VEC_EQ((vector<int8_t>{-1, 2, 3, 4}), read_vector<int8_t>(r));
        unsetenv("NGRAPH_PASS_ENABLES");
    }
}

GPU_TEST(HIP, quant_fusion_qconvb_add)
{
    for (bool signed_summand : {true, false})
        for (bool through_reshape : {false, true})
        {
            vector<vector<float>> args{ramp(8, 2.0f, 1, 6), ramp(2, 2.0f, -2, 3), ramp(1, 4.0f, 2, 2), ramp(4, 4.0f, signed_summand ? -9 : 0, 9)}; // summand: multiples of the output scale, so the fused sum stays exact
            auto off = execute(make_qconvb_add(signed_summand, through_reshape), args, false);
            auto on = execute(make_qconvb_add(signed_summand, through_reshape), args, true);
            EXPECT_VEC_EQ(off.at(0), on.at(0));
        }
}
