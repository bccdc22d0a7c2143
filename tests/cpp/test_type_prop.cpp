// Validation and type / shape inference of the quantized ops, written after the reference's
// test/type_prop/{quantize,dequantize,quantized_convolution,quantized_dot}.cpp: same constructor
// arguments, same expected message fragments.  Needs no GPU.
#include "test_util.hpp"

using namespace std;
using namespace ngraph;

#define EXPECT_VALIDATION_FAILURE(stmt, fragment)                                                  \
    do                                                                                             \
    {                                                                                              \
        bool ok_ = false;                                                                          \
        try                                                                                        \
        {                                                                                          \
            stmt;                                                                                  \
        }                                                                                          \
        catch (const NodeValidationFailure& error)                                                 \
        {                                                                                          \
            ok_ = string(error.what()).find(fragment) != string::npos;                             \
            if (!ok_)                                                                              \
                mini_test::fail(__FILE__, __LINE__, string("message '") + error.what() + "' lacks '" + fragment + "'");         \
        }                                                                                          \
        catch (...)                                                                                \
        {                                                                                          \
        }                                                                                          \
        if (!ok_)                                                                                  \
            mini_test::fail(__FILE__, __LINE__, "expected NodeValidationFailure: " fragment);      \
    } while (0)

namespace
{
    const auto RTI = op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_INFINITY;

    shared_ptr<Node> quantize(element::Type batch_t, Shape batch, element::Type scale_t, Shape scale, element::Type zp_t, Shape zp,
                              element::Type out_t, AxisSet axes)
    {
        return make_shared<op::v0::Quantize>(make_shared<op::v0::Parameter>(batch_t, batch), make_shared<op::v0::Parameter>(scale_t, scale),
                                             make_shared<op::v0::Parameter>(zp_t, zp), out_t, axes, RTI);
    }
    shared_ptr<Node> dequantize(element::Type batch_t, Shape batch, element::Type scale_t, Shape scale, element::Type zp_t, Shape zp,
                                element::Type out_t, AxisSet axes)
    {
        return make_shared<op::v0::Dequantize>(make_shared<op::v0::Parameter>(batch_t, batch), make_shared<op::v0::Parameter>(scale_t, scale),
                                               make_shared<op::v0::Parameter>(zp_t, zp), out_t, axes);
    }
}

CPU_TEST(type_prop, quantize_ok_cases)
{
    Shape batch{64, 3, 480, 640};
    // per channel, per image, per row, per image+channel, whole batch
    struct
    {
        Shape so;
        AxisSet axes;
    } cases[] = {{Shape{3}, AxisSet{1}}, {Shape{64}, AxisSet{0}}, {Shape{480}, AxisSet{2}}, {Shape{64, 3}, AxisSet{0, 1}}, {Shape{}, AxisSet{}}};
    for (auto& c : cases)
    {
        auto q = quantize(element::f32, batch, element::f32, c.so, element::i8, c.so, element::i8, c.axes);
        EXPECT_EQ(q->get_output_element_type(0), element::i8);
        EXPECT_EQ(q->get_output_shape(0), batch);
    }
    EXPECT_EQ(quantize(element::f64, batch, element::f64, Shape{}, element::i8, Shape{}, element::i8, AxisSet{})->get_output_element_type(0), element::i8);
    EXPECT_EQ(quantize(element::f64, batch, element::f64, Shape{}, element::u8, Shape{}, element::u8, AxisSet{})->get_output_element_type(0), element::u8);
}

CPU_TEST(type_prop, quantize_failures)
{
    Shape batch{64, 3, 480, 640};
    EXPECT_VALIDATION_FAILURE(quantize(element::f64, batch, element::f64, Shape{}, element::dynamic, Shape{}, element::dynamic, AxisSet{}),
                              "Output element type must not be dynamic");
    EXPECT_VALIDATION_FAILURE(quantize(element::i8, batch, element::i8, Shape{}, element::u8, Shape{}, element::u8, AxisSet{}),
                              "Scale / input element type (i8) must be a floating point number");
    EXPECT_VALIDATION_FAILURE(quantize(element::f32, batch, element::f32, Shape{}, element::f32, Shape{}, element::f32, AxisSet{}),
                              "Output element type (f32) must be a quantized type");
    EXPECT_VALIDATION_FAILURE(quantize(element::f32, batch, element::f64, Shape{}, element::i8, Shape{}, element::i8, AxisSet{}),
                              "Scale element type (f64) must match input element type (f32)");
    EXPECT_VALIDATION_FAILURE(quantize(element::f32, batch, element::f32, Shape{}, element::u8, Shape{}, element::i8, AxisSet{}),
                              "Zero point element type (u8) must match output element type (i8)");
    EXPECT_VALIDATION_FAILURE(quantize(element::f32, batch, element::f32, Shape{320}, element::i8, Shape{320}, element::i8, AxisSet{3, 4}),
                              "Quantization axis (4) must be less than input shape rank (4)");
    EXPECT_VALIDATION_FAILURE(quantize(element::f32, batch, element::f32, Shape{64, 4}, element::i8, Shape{64, 3}, element::i8, AxisSet{0, 1}),
                              "Scale shape ({64,4}) and zero point shape ({64,3}) must match");
    EXPECT_VALIDATION_FAILURE(quantize(element::f32, batch, element::f32, Shape{64, 3, 2}, element::i8, Shape{64, 3}, element::i8, AxisSet{0, 1}),
                              "Scale shape ({64,3,2}) and zero point shape ({64,3}) must match");
    EXPECT_VALIDATION_FAILURE(quantize(element::f32, batch, element::f32, Shape{64, 3}, element::i8, Shape{64, 4}, element::i8, AxisSet{0, 1}),
                              "Scale shape ({64,3}) and zero point shape ({64,4}) must match");
    EXPECT_VALIDATION_FAILURE(quantize(element::f32, batch, element::f32, Shape{64, 3, 2}, element::i8, Shape{64, 3, 2}, element::i8, AxisSet{0, 1}),
                              "Scale / zero point rank (3) does not match the number of quantization axes (2)");
}

CPU_TEST(type_prop, dequantize_ok_and_failures)
{
    Shape batch{64, 3, 480, 640};
    auto d = dequantize(element::i8, batch, element::f32, Shape{3}, element::i8, Shape{3}, element::f32, AxisSet{1});
    EXPECT_EQ(d->get_output_element_type(0), element::f32);
    EXPECT_EQ(d->get_output_shape(0), batch);
    EXPECT_EQ(dequantize(element::u8, batch, element::f64, Shape{}, element::u8, Shape{}, element::f64, AxisSet{})->get_output_element_type(0), element::f64);
    EXPECT_VALIDATION_FAILURE(dequantize(element::i8, batch, element::f32, Shape{}, element::i8, Shape{}, element::dynamic, AxisSet{}),
                              "Output element type must not be dynamic");
    EXPECT_VALIDATION_FAILURE(dequantize(element::i8, batch, element::i8, Shape{}, element::i8, Shape{}, element::i8, AxisSet{}),
                              "Output element type (i8) must be a floating point type");
    EXPECT_VALIDATION_FAILURE(dequantize(element::f32, batch, element::f32, Shape{}, element::f32, Shape{}, element::f32, AxisSet{}),
                              "Zero point / input element type (f32) must be a quantized type");
    EXPECT_VALIDATION_FAILURE(dequantize(element::i8, batch, element::f64, Shape{}, element::i8, Shape{}, element::f32, AxisSet{}),
                              "Scale element type (f64) must match output element type (f32)");
    EXPECT_VALIDATION_FAILURE(dequantize(element::i8, batch, element::f32, Shape{}, element::u8, Shape{}, element::f32, AxisSet{}),
                              "Zero point element type (u8) must match input element type (i8)");
    EXPECT_VALIDATION_FAILURE(dequantize(element::i8, batch, element::f32, Shape{320}, element::i8, Shape{320}, element::f32, AxisSet{3, 4}),
                              "Quantization axis (4) must be less than input shape rank (4)");
    EXPECT_VALIDATION_FAILURE(dequantize(element::i8, batch, element::f32, Shape{64, 3}, element::i8, Shape{64, 3, 2}, element::f32, AxisSet{0, 1}),
                              "Scale shape ({64,3}) and zero point shape ({64,3,2}) must match");
}

namespace
{
    struct ConvArgs
    {
        element::Type input_t = element::u8, filter_t = element::i8, output_t = element::i8;
        element::Type scale_t = element::f32, input_zp_t = element::u8, filter_zp_t = element::i8, output_zp_t = element::i8;
        Shape input_zp_shape{}, filter_zp_shape{}, output_zp_shape{};
        AxisSet input_axes{}, filter_axes{}, output_axes{};
    };

    shared_ptr<Node> qconv(const ConvArgs& a)
    {
        auto batch = make_shared<op::v0::Parameter>(a.input_t, Shape{64, 3, 100});
        auto filter = make_shared<op::v0::Parameter>(a.filter_t, Shape{128, 3, 10});
        auto scale = make_shared<op::v0::Parameter>(a.scale_t, Shape{});
        auto izp = make_shared<op::v0::Parameter>(a.input_zp_t, a.input_zp_shape);
        auto fzp = make_shared<op::v0::Parameter>(a.filter_zp_t, a.filter_zp_shape);
        auto ozp = make_shared<op::v0::Parameter>(a.output_zp_t, a.output_zp_shape);
        return make_shared<op::v0::QuantizedConvolution>(batch, filter, Strides{1}, Strides{1}, CoordinateDiff{0}, CoordinateDiff{0}, Strides{1},
                                                         scale, izp, scale, fzp, scale, ozp, a.output_t, a.input_axes, a.filter_axes,
                                                         a.output_axes);
    }
}

CPU_TEST(type_prop, quantized_conv)
{
    ConvArgs ok;
    auto q = qconv(ok);
    EXPECT_EQ(q->get_element_type(), element::i8);
    EXPECT_EQ(q->get_shape(), (Shape{64, 128, 91}));
    ConvArgs ok32 = ok;
    ok32.output_t = ok32.output_zp_t = element::i32;
    EXPECT_EQ(qconv(ok32)->get_element_type(), element::i32);

    ConvArgs a = ok;
    a.input_t = a.input_zp_t = element::f32;
    EXPECT_VALIDATION_FAILURE(qconv(a), "Input element type (f32) must be a quantized type");
    a = ok;
    a.filter_t = a.filter_zp_t = element::f32;
    EXPECT_VALIDATION_FAILURE(qconv(a), "Filter element type (f32) must be a quantized type");
    a = ok;
    a.output_t = element::dynamic;
    EXPECT_VALIDATION_FAILURE(qconv(a), "Output element type must not be dynamic");
    a = ok;
    a.scale_t = element::i8;
    EXPECT_VALIDATION_FAILURE(qconv(a), "Scale must be a floating point number");
    a = ok;
    a.input_zp_t = element::i8;
    EXPECT_VALIDATION_FAILURE(qconv(a), "Input Zero point element type (i8) must match input element type (u8)");
    a = ok;
    a.filter_zp_t = element::u8;
    EXPECT_VALIDATION_FAILURE(qconv(a), "Filter Zero point element type (u8) must match filter element type (i8)");
    a = ok;
    a.input_zp_shape = Shape{1, 2};
    EXPECT_VALIDATION_FAILURE(qconv(a), "Input scale and input zero point shape must be same and 1");
    a = ok;
    a.filter_zp_shape = Shape{1, 2};
    EXPECT_VALIDATION_FAILURE(qconv(a), "Filter scale and filter zero point shape must be same and 1");
    a = ok;
    a.output_zp_shape = Shape{1, 2};
    EXPECT_VALIDATION_FAILURE(qconv(a), "Output scale and output zero point shape must be same and 1");
    for (int which = 0; which < 3; ++which)
    {
        a = ok;
        (which == 0 ? a.input_axes : which == 1 ? a.filter_axes : a.output_axes) = AxisSet{1};
        EXPECT_VALIDATION_FAILURE(qconv(a), "Input, filter and output AxisSet should be empty");
    }
}

namespace
{
    struct DotArgs
    {
        element::Type input0_t = element::u8, input1_t = element::i8, output_t = element::i8;
        element::Type scale_t = element::f32, zp0_t = element::u8, zp1_t = element::i8, ozp_t = element::i8;
        Shape zp0_shape{}, zp1_shape{}, ozp_shape{};
        AxisSet axes0{}, axes1{}, axes_out{};
    };
    shared_ptr<Node> qdot(const DotArgs& a)
    {
        auto in0 = make_shared<op::v0::Parameter>(a.input0_t, Shape{64});
        auto in1 = make_shared<op::v0::Parameter>(a.input1_t, Shape{64});
        auto scale = make_shared<op::v0::Parameter>(a.scale_t, Shape{});
        auto zp0 = make_shared<op::v0::Parameter>(a.zp0_t, a.zp0_shape);
        auto zp1 = make_shared<op::v0::Parameter>(a.zp1_t, a.zp1_shape);
        auto ozp = make_shared<op::v0::Parameter>(a.ozp_t, a.ozp_shape);
        return make_shared<op::v0::QuantizedDot>(in0, in1, 1, scale, zp0, scale, zp1, scale, ozp, a.output_t, a.axes0, a.axes1, a.axes_out);
    }
}

CPU_TEST(type_prop, quantized_dot)
{
    DotArgs ok;
    auto q = qdot(ok);
    EXPECT_EQ(q->get_element_type(), element::i8);
    EXPECT_EQ(q->get_shape(), Shape{});
    DotArgs ok32 = ok;
    ok32.output_t = ok32.ozp_t = element::i32;
    EXPECT_EQ(qdot(ok32)->get_element_type(), element::i32);

    DotArgs a = ok;
    a.input0_t = a.zp0_t = element::f32;
    EXPECT_VALIDATION_FAILURE(qdot(a), "Input0 element type (f32) must be a quantized type");
    a = ok;
    a.input1_t = a.zp1_t = element::f32;
    EXPECT_VALIDATION_FAILURE(qdot(a), "Input1 element type (f32) must be a quantized type");
    a = ok;
    a.output_t = element::dynamic;
    EXPECT_VALIDATION_FAILURE(qdot(a), "Output element type must not be dynamic");
    a = ok;
    a.scale_t = element::i8;
    EXPECT_VALIDATION_FAILURE(qdot(a), "Scale must be a floating point number");
    a = ok;
    a.zp0_t = element::i8;
    EXPECT_VALIDATION_FAILURE(qdot(a), "Input0 Zero point element type (i8) must match input0 element type (u8)");
    a = ok;
    a.zp1_t = element::u8;
    EXPECT_VALIDATION_FAILURE(qdot(a), "Input1 Zero point element type (u8) must match input1 element type (i8)");
    a = ok;
    a.zp0_shape = Shape{1, 2};
    EXPECT_VALIDATION_FAILURE(qdot(a), "Input0 scale and input0 zero point shape must be same and 1");
    a = ok;
    a.zp1_shape = Shape{1, 2};
    EXPECT_VALIDATION_FAILURE(qdot(a), "Input1 scale and input1 zero point shape must be same and 1");
    a = ok;
    a.ozp_shape = Shape{1, 2};
    EXPECT_VALIDATION_FAILURE(qdot(a), "Output scale and output zero point shape must be same and 1");
    for (int which = 0; which < 3; ++which)
    {
        a = ok;
        (which == 0 ? a.axes0 : which == 1 ? a.axes1 : a.axes_out) = AxisSet{1};
        EXPECT_VALIDATION_FAILURE(qdot(a), "Input0, input1 and output AxisSet should be empty");
    }
}

CPU_TEST(type_prop, fused_ops_output_types)
{
    auto data = make_shared<op::v0::Parameter>(element::u8, Shape{1, 16, 8, 8});
    auto filt = make_shared<op::v0::Parameter>(element::i8, Shape{32, 16, 3, 3});
    auto bias = make_shared<op::v0::Parameter>(element::i32, Shape{32});
    auto scale = make_shared<op::v0::Parameter>(element::f32, Shape{});
    auto sum_u = make_shared<op::v0::Parameter>(element::u8, Shape{1, 32, 8, 8});
    auto sum_i = make_shared<op::v0::Parameter>(element::i8, Shape{1, 32, 8, 8});
    Strides one{1, 1};
    CoordinateDiff pad{1, 1};
    auto b0 = make_shared<op::v0::QuantizedConvolutionBias>(data, filt, bias, one, one, pad, pad, one, scale, false);
    auto b1 = make_shared<op::v0::QuantizedConvolutionBias>(data, filt, bias, one, one, pad, pad, one, scale, true);
    EXPECT_EQ(b0->get_element_type(), element::i8);
    EXPECT_EQ(b1->get_element_type(), element::u8);
    EXPECT_EQ(b1->get_shape(), (Shape{1, 32, 8, 8}));
    EXPECT_EQ(make_shared<op::v0::QuantizedConvolutionRelu>(data, filt, one, one, pad, pad, one, scale)->get_element_type(), element::u8);
    EXPECT_EQ(make_shared<op::v0::QuantizedConvolutionBiasAdd>(data, filt, bias, sum_u, one, one, pad, pad, one, scale, scale, true)->get_element_type(), element::u8);
    // the signed variant stays i8 even with relu
    EXPECT_EQ(make_shared<op::v0::QuantizedConvolutionBiasSignedAdd>(data, filt, bias, sum_i, one, one, pad, pad, one, scale, scale, true)->get_element_type(), element::i8);
    auto a = make_shared<op::v0::Parameter>(element::u8, Shape{4, 3});
    auto w = make_shared<op::v0::Parameter>(element::i8, Shape{5, 3});
    auto wb = make_shared<op::v0::Parameter>(element::i32, Shape{5});
    EXPECT_EQ(make_shared<op::v0::QuantizedDotBias>(a, w, wb, scale, false, false)->get_element_type(), element::f32);
    EXPECT_EQ(make_shared<op::v0::QuantizedDotBias>(a, w, wb, scale, true, false)->get_element_type(), element::i8);
    EXPECT_EQ(make_shared<op::v0::QuantizedDotBias>(a, w, wb, scale, true, true)->get_element_type(), element::u8);
    EXPECT_EQ(make_shared<op::v0::QuantizedDotBias>(a, w, wb, scale, true, true)->get_shape(), (Shape{4, 5}));
    auto w_bad = make_shared<op::v0::Parameter>(element::i8, Shape{5, 4});
    EXPECT_THROW(make_shared<op::v0::QuantizedDotBias>(a, w_bad, wb, scale), NodeValidationFailure);
}

CPU_TEST(builder, scale_subgraph_constant_folds)
{
    // get_scale(0, 255, u8) == 1, get_scale(22, 90, i8) == 90/127, the (is * fs / os) of the conv builders
    auto c = [](float v) { return op::v0::Constant::create(element::f32, Shape{}, {v}); };
    auto data = make_shared<op::v0::Parameter>(element::u8, Shape{1, 1, 3, 4});
    auto filt = make_shared<op::v0::Parameter>(element::i8, Shape{1, 1, 3, 3});
    auto cv = builder::QuantizedConvolutionReluBuilder(data, filt, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1},
                                                       Strides{1, 1}, c(0), c(255), c(-127), c(127), c(22), c(90));
    auto f = make_shared<Function>(cv, ParameterVector{data, filt});
    size_t before = f->get_ordered_ops().size();
    constant_fold(f);
    auto ops = f->get_ordered_ops();
    EXPECT_TRUE(ops.size() < before);
    EXPECT_EQ(ops.size(), 5u); // data, filter, folded scale, conv, result
    auto folded = as_type_ptr<op::v0::Constant>(f->get_results()[0]->get_argument(0)->get_argument(2));
    EXPECT_TRUE(folded != nullptr);
    if (folded)
    {
        float expected = (255.0f / 255.0f) * (127.0f / 127.0f) / (90.0f / 255.0f);
        EXPECT_EQ(folded->get_vector<float>()[0], expected);
    }
    // clone_function yields an independent, equal graph
    auto g = clone_function(*f);
    EXPECT_EQ(g->get_ordered_ops().size(), ops.size());
    EXPECT_TRUE(g->get_parameters()[0] != f->get_parameters()[0]);
}
