// The quantized ops through the backend, written after the reference's
// test/backend/quantized_convolution.in.cpp:31-134, test/backend/quantized_dot.in.cpp:31-115,
// test/backend/quantize_dequantize.in.cpp (all 28 vectors, table-driven) and
// test/builder_quantization.cpp:51-847,995-1098 (which the reference can only run on its CPU
// backend), against backend "HIP".
#include "test_util.hpp"

using namespace std;
using namespace ngraph;

GPU_TEST(HIP, quantized_convolution)
{
    Shape shape_a{1, 1, 3, 4};
    Shape shape_b{1, 1, 3, 3};
    Shape shape_r{1, 1, 3, 4};
    vector<uint8_t> a_data = {1, 2, 3, 4, 5, 6, 7, 0, 1, 2, 3, 4};
    vector<int8_t> b_data = {1, 2, 3, 4, 5, 0, 0, 1, 2};
    auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto B = make_shared<op::v0::Parameter>(element::i8, shape_b);
    ParameterVector ranges;
    for (int i = 0; i < 6; ++i)
        ranges.push_back(make_shared<op::v0::Parameter>(element::f32, Shape{}));
    auto CV = builder::QuantizedConvolutionBuilder(A, B, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1}, Strides{1, 1},
                                                   ranges[0], ranges[1], ranges[2], ranges[3], ranges[4], ranges[5], element::i8);
    ParameterVector params{A, B};
    params.insert(params.end(), ranges.begin(), ranges.end());
    auto f = make_shared<Function>(OutputVector{CV}, params);
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor(element::u8, shape_a);
    copy_data(a, a_data);
    auto b = backend->create_tensor(element::i8, shape_b);
    copy_data(b, b_data);
    vector<shared_ptr<runtime::Tensor>> inputs{a, b};
    for (float v : {0.0f, 255.0f, -127.0f, 127.0f, 22.0f, 90.0f})
    {
        auto t = backend->create_tensor(element::f32, Shape{});
        copy_data(t, vector<float>{v});
        inputs.push_back(t);
    }
    auto result = backend->create_tensor(element::i8, shape_r);
    auto handle = backend->compile(f);
    handle->call_with_validate({result}, inputs);
    EXPECT_VEC_EQ((vector<int8_t>{31, 48, 42, 45, 54, 102, 127, 61, 47, 73, 61, 55}), read_vector<int8_t>(result));
}

GPU_TEST(HIP, quantized_conv_int32_output)
{
    Shape shape_a{1, 1, 3, 4};
    Shape shape_b{1, 1, 3, 3};
    Shape shape_r{1, 1, 3, 4};
    vector<uint8_t> a_data = {1, 2, 3, 4, 5, 6, 7, 0, 1, 2, 3, 4};
    vector<uint8_t> b_data = {1, 2, 3, 4, 5, 0, 0, 1, 2};
    auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto B = make_shared<op::v0::Parameter>(element::u8, shape_b);
    auto C = make_shared<op::v0::Parameter>(element::f32, Shape{});
    auto D = op::v0::Constant::create(element::u8, Shape{}, {0});
    auto E = make_shared<op::v0::Parameter>(element::f32, Shape{});
    auto F = op::v0::Constant::create(element::u8, Shape{}, {0});
    auto G = make_shared<op::v0::Parameter>(element::f32, Shape{});
    auto H = op::v0::Constant::create(element::i32, Shape{}, {0});
    auto CV = make_shared<op::v0::QuantizedConvolution>(A, B, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1},
                                                        Strides{1, 1}, C, D, E, F, G, H, element::i32);
    auto f = make_shared<Function>(OutputVector{CV}, ParameterVector{A, B, C, E, G});
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor(element::u8, shape_a);
    copy_data(a, a_data);
    auto b = backend->create_tensor(element::u8, shape_b);
    copy_data(b, b_data);
    auto c = backend->create_tensor(element::f32, Shape{});
    copy_data(c, vector<float>{1.0f});
    auto d = backend->create_tensor(element::f32, Shape{});
    copy_data(d, vector<float>{1.0f});
    auto e = backend->create_tensor(element::f32, Shape{});
    copy_data(e, vector<float>{1.0f});
    auto result = backend->create_tensor(element::i32, shape_r);
    auto handle = backend->compile(f);
    handle->call_with_validate({result}, {a, b, c, d, e});
    EXPECT_VEC_EQ((vector<int32_t>{22, 34, 30, 32, 38, 72, 90, 43, 33, 52, 43, 39}), read_vector<int32_t>(result));
}

// a constant i8 filter with constant zero zero-points takes the prepacked MFMA path at compile time
GPU_TEST(HIP, quantized_convolution_constant_filter_mfma)
{
    Shape shape_a{1, 16, 5, 5};
    Shape shape_b{8, 16, 3, 3};
    vector<uint8_t> a_data(16 * 25);
    for (size_t i = 0; i < a_data.size(); ++i)
        a_data[i] = static_cast<uint8_t>((i * 37 + 11) % 256);
    vector<int8_t> b_data(8 * 16 * 9);
    for (size_t i = 0; i < b_data.size(); ++i)
        b_data[i] = static_cast<int8_t>(static_cast<int>((i * 53 + 7) % 255) - 127);
    auto make = [&](bool constant_filter) {
        auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
        shared_ptr<Node> B;
        ParameterVector params{A};
        if (constant_filter)
            B = op::v0::Constant::create(element::i8, shape_b, b_data);
        else
        {
            auto P = make_shared<op::v0::Parameter>(element::i8, shape_b);
            params.push_back(P);
            B = P;
        }
        auto one = op::v0::Constant::create(element::f32, Shape{}, {1.0f});
        auto zu = op::v0::Constant::create(element::u8, Shape{}, {0});
        auto zi = op::v0::Constant::create(element::i8, Shape{}, {0});
        auto z32 = op::v0::Constant::create(element::i32, Shape{}, {0});
        auto CV = make_shared<op::v0::QuantizedConvolution>(A, B, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1},
                                                            Strides{1, 1}, one, zu, one, zi, one, z32, element::i32);
        return make_shared<Function>(OutputVector{CV}, params);
    };
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor(element::u8, shape_a);
    copy_data(a, a_data);
    auto b = backend->create_tensor(element::i8, shape_b);
    copy_data(b, b_data);
    auto r1 = backend->create_tensor(element::i32, Shape{1, 8, 5, 5});
    auto r2 = backend->create_tensor(element::i32, Shape{1, 8, 5, 5});
    backend->compile(make(true))->call_with_validate({r1}, {a});
    backend->compile(make(false))->call_with_validate({r2}, {a, b});
    auto v1 = read_vector<int32_t>(r1);
    EXPECT_VEC_EQ(v1, read_vector<int32_t>(r2));
    // one accumulator by hand: output (k=0, y=0, x=0)
    int32_t acc = 0;
    for (int c = 0; c < 16; ++c)
        for (int r = 1; r < 3; ++r)
            for (int s = 1; s < 3; ++s)
                acc += static_cast<int32_t>(a_data[(c * 5 + (r - 1)) * 5 + (s - 1)]) * b_data[(c * 3 + r) * 3 + s];
    EXPECT_EQ(v1[0], acc);
}

GPU_TEST(HIP, quantized_dot_u8u8)
{
    Shape shape_a{1, 2};
    vector<uint8_t> a_data = {2, 3};
    Shape shape_b{2, 3};
    vector<uint8_t> b_data = {0, 2, 4, 1, 3, 5};
    auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto B = make_shared<op::v0::Parameter>(element::u8, shape_b);
    auto input_scale = op::v0::Constant::create(element::f32, Shape{}, {2});
    auto input_zero_point = op::v0::Constant::create(element::u8, Shape{}, {0});
    auto filter_scale = op::v0::Constant::create(element::f32, Shape{}, {1});
    auto filter_zero_point = op::v0::Constant::create(element::u8, Shape{}, {0});
    auto output_scale = op::v0::Constant::create(element::f32, Shape{}, {2});
    auto output_zero_point = op::v0::Constant::create(element::u8, Shape{}, {0});
    AxisSet axes{};
    Shape shape_r{1, 3};
    auto QD = make_shared<op::v0::QuantizedDot>(A, B, 1, input_scale, input_zero_point, filter_scale, filter_zero_point, output_scale,
                                                output_zero_point, element::u8, axes, axes, axes);
    auto f = make_shared<Function>(OutputVector{QD}, ParameterVector{A, B});
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor(element::u8, shape_a);
    copy_data(a, a_data);
    auto b = backend->create_tensor(element::u8, shape_b);
    copy_data(b, b_data);
    auto result = backend->create_tensor(element::u8, shape_r);
    auto handle = backend->compile(f);
    handle->call_with_validate({result}, {a, b});
    EXPECT_VEC_EQ((vector<uint8_t>{3, 13, 23}), read_vector<uint8_t>(result));
}

GPU_TEST(HIP, quantized_dot_int32_output)
{
    Shape shape_a{1, 2};
    vector<uint8_t> a_data = {2, 3};
    Shape shape_b{2, 3};
    vector<int8_t> b_data = {0, 1, 2, 3, 4, 5};
    auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto B = make_shared<op::v0::Parameter>(element::i8, shape_b);
    auto one = op::v0::Constant::create(element::f32, Shape{}, {1});
    auto zu = op::v0::Constant::create(element::u8, Shape{}, {0});
    auto zi = op::v0::Constant::create(element::i8, Shape{}, {0});
    auto z32 = op::v0::Constant::create(element::i32, Shape{}, {0});
    AxisSet axes{};
    auto QD = make_shared<op::v0::QuantizedDot>(A, B, 1, one, zu, one, zi, one, z32, element::i32, axes, axes, axes);
    auto f = make_shared<Function>(OutputVector{QD}, ParameterVector{A, B});
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor(element::u8, shape_a);
    copy_data(a, a_data);
    auto b = backend->create_tensor(element::i8, shape_b);
    copy_data(b, b_data);
    auto result = backend->create_tensor(element::i32, Shape{1, 3});
    auto handle = backend->compile(f);
    handle->call_with_validate({result}, {a, b});
    EXPECT_VEC_EQ((vector<int32_t>{9, 14, 19}), read_vector<int32_t>(result));
}

// ------------------------------------------------------------------ quantize / dequantize (28 vectors)
namespace
{
    struct QdqCase
    {
        const char* name;
        bool quantize;
        const char* in_t;
        const char* out_t;
        vector<size_t> shape;
        vector<size_t> axes;
        op::v0::Quantize::RoundMode mode;
        vector<double> scale, offset, input, expected;
        bool dynamic;
    };
    const vector<QdqCase> qdq_cases = {
#include "qdq_table.inc"
    };

    element::Type type_named(const string& n)
    {
        if (n == "f32")
            return element::f32;
        if (n == "f64")
            return element::f64;
        if (n == "u8")
            return element::u8;
        if (n == "i8")
            return element::i8;
        return element::i32;
    }

    // host <-> tensor with values carried as double
    void write_as(const shared_ptr<runtime::Tensor>& t, const vector<double>& v)
    {
        auto c = op::v0::Constant::create(t->get_element_type(), t->get_shape(), v);
        t->write(c->get_data_ptr(), t->get_size_in_bytes());
    }
    vector<double> read_as(const shared_ptr<runtime::Tensor>& t)
    {
        vector<uint8_t> bytes(t->get_size_in_bytes());
        t->read(bytes.data(), bytes.size());
        return op::v0::Constant(t->get_element_type(), t->get_shape(), bytes.data()).get_values_as_double();
    }
}

GPU_TEST(HIP, quantize_dequantize_vectors)
{
    auto backend = runtime::Backend::create("HIP");
    EXPECT_EQ(qdq_cases.size(), 28u);
    for (const auto& c : qdq_cases)
    {
        const element::Type in_t = type_named(c.in_t), out_t = type_named(c.out_t);
        const element::Type real_t = c.quantize ? in_t : out_t, quant_t = c.quantize ? out_t : in_t;
        Shape shape(c.shape), so_shape;
        AxisSet axes;
        for (size_t a : c.axes)
        {
            axes.insert(a);
            so_shape.push_back(shape[a]);
        }
        auto X = make_shared<op::v0::Parameter>(in_t, shape);
        ParameterVector params{X};
        shared_ptr<Node> scale, offset;
        if (c.dynamic)
        {
            auto S = make_shared<op::v0::Parameter>(real_t, so_shape);
            auto O = make_shared<op::v0::Parameter>(quant_t, so_shape);
            params.push_back(S);
            params.push_back(O);
            scale = S;
            offset = O;
        }
        else
        {
            scale = op::v0::Constant::create(real_t, so_shape, c.scale);
            offset = op::v0::Constant::create(quant_t, so_shape, c.offset);
        }
        shared_ptr<Node> op;
        if (c.quantize)
            op = make_shared<op::v0::Quantize>(X, scale, offset, out_t, axes, c.mode);
        else
            op = make_shared<op::v0::Dequantize>(X, scale, offset, out_t, axes);
        auto f = make_shared<Function>(op, params);
        auto x = backend->create_tensor(in_t, shape);
        auto y = backend->create_tensor(out_t, shape);
        write_as(x, c.input);
        vector<shared_ptr<runtime::Tensor>> inputs{x};
        if (c.dynamic)
        {
            auto s = backend->create_tensor(real_t, so_shape);
            auto o = backend->create_tensor(quant_t, so_shape);
            write_as(s, c.scale);
            write_as(o, c.offset);
            inputs.push_back(s);
            inputs.push_back(o);
        }
        backend->compile(f)->call_with_validate({y}, inputs);
        auto got = read_as(y);
        if (!(got == c.expected))
            mini_test::fail(__FILE__, __LINE__, string(c.name) + ": expected " + mini_test::show(c.expected) + " got " + mini_test::show(got));
    }
}

// ------------------------------------------------------------------ builder tests
namespace
{
    shared_ptr<Node> scalar(float v, bool rank1 = false) { return op::v0::Constant::create(element::f32, rank1 ? Shape{1} : Shape{}, {v}); }

    template <typename T>
    shared_ptr<runtime::Tensor> tensor_of(const shared_ptr<runtime::Backend>& b, const element::Type& t, const Shape& s, const vector<T>& v)
    {
        auto x = b->create_tensor(t, s);
        copy_data(x, v);
        return x;
    }
}

GPU_TEST(builder, scaled_QC_with_relu)
{
    Shape shape_a{1, 1, 3, 3}, shape_b{1, 1, 3, 3}, shape_r{1, 1, 3, 3};
    vector<uint8_t> a_data = {1, 2, 3, 4, 5, 6, 7, 8, 9};
    vector<int8_t> b_data = {1, 2, 1, 0, 0, 0, -1, -2, -1};
    auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto B = make_shared<op::v0::Parameter>(element::i8, shape_b);
    auto CV = builder::QuantizedConvolutionReluBuilder(A, B, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1}, Strides{1, 1},
                                                       scalar(0.0f, true), scalar(255.0f, true), scalar(-127.0f, true), scalar(127.0f, true),
                                                       scalar(20.0f, true), scalar(-24.0f, true));
    auto f = make_shared<Function>(OutputVector{CV}, ParameterVector{A, B});
    constant_fold(f);
    auto backend = runtime::Backend::create("HIP");
    auto a = tensor_of(backend, element::u8, shape_a, a_data);
    auto b = tensor_of(backend, element::i8, shape_b, b_data);
    auto result = backend->create_tensor(element::u8, shape_r);
    backend->compile(f)->call_with_validate({result}, {a, b});
    EXPECT_VEC_EQ((vector<uint8_t>{0, 0, 0, 0, 0, 0, 138, 212, 181}), read_vector<uint8_t>(result));
}

GPU_TEST(builder, dynamic_scaled_QC_with_relu)
{
    Shape shape_a{1, 1, 3, 3}, shape_b{1, 1, 3, 3}, shape_r{1, 1, 3, 3};
    auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto B = make_shared<op::v0::Parameter>(element::i8, shape_b);
    ParameterVector r;
    for (int i = 0; i < 6; ++i)
        r.push_back(make_shared<op::v0::Parameter>(element::f32, Shape{1}));
    auto CV = builder::QuantizedConvolutionReluBuilder(A, B, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1}, Strides{1, 1},
                                                       r[0], r[1], r[2], r[3], r[4], r[5]);
    ParameterVector params{A, B};
    params.insert(params.end(), r.begin(), r.end());
    auto f = make_shared<Function>(OutputVector{CV}, params);
    auto backend = runtime::Backend::create("HIP");
    vector<shared_ptr<runtime::Tensor>> in{tensor_of(backend, element::u8, shape_a, vector<uint8_t>{1, 2, 3, 4, 5, 6, 7, 8, 9}),
                                           tensor_of(backend, element::i8, shape_b, vector<int8_t>{1, 2, 1, 0, 0, 0, -1, -2, -1})};
    for (float v : {0.0f, 255.0f, -127.0f, 127.0f, 20.0f, -24.0f})
        in.push_back(tensor_of(backend, element::f32, Shape{1}, vector<float>{v}));
    auto result = backend->create_tensor(element::u8, shape_r);
    backend->compile(f)->call_with_validate({result}, in);
    EXPECT_VEC_EQ((vector<uint8_t>{0, 0, 0, 0, 0, 0, 138, 212, 181}), read_vector<uint8_t>(result));
}

GPU_TEST(builder, scaled_QC_with_bias)
{
    Shape shape_a{1, 1, 3, 4}, shape_b{1, 1, 3, 3}, shape_r{1, 1, 3, 4};
    auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto B = make_shared<op::v0::Parameter>(element::i8, shape_b);
    auto Bias = make_shared<op::v0::Parameter>(element::i32, Shape{1});
    auto CV = builder::QuantizedConvolutionBiasBuilder(A, B, Bias, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1},
                                                       Strides{1, 1}, scalar(0.0f, true), scalar(255.0f, true), scalar(-127.0f, true),
                                                       scalar(127.0f, true), scalar(22.0f, true), scalar(90.0f, true));
    auto f = make_shared<Function>(OutputVector{CV}, ParameterVector{A, B, Bias});
    constant_fold(f);
    auto backend = runtime::Backend::create("HIP");
    auto a = tensor_of(backend, element::u8, shape_a, vector<uint8_t>{1, 2, 3, 4, 5, 6, 7, 0, 1, 2, 3, 4});
    auto b = tensor_of(backend, element::i8, shape_b, vector<int8_t>{1, 2, 3, 4, 5, 0, 0, 1, 2});
    auto c = tensor_of(backend, element::i32, Shape{1}, vector<int32_t>{5});
    auto result = backend->create_tensor(element::i8, shape_r);
    backend->compile(f)->call_with_validate({result}, {a, b, c});
    EXPECT_VEC_EQ((vector<int8_t>{38, 55, 49, 52, 61, 109, 127, 68, 54, 80, 68, 62}), read_vector<int8_t>(result));
}

GPU_TEST(builder, scaled_QC_with_bias_and_relu_and_f32_bias)
{
    Shape shape_a{1, 1, 3, 3}, shape_b{1, 1, 3, 3}, shape_r{1, 1, 3, 3};
    auto backend = runtime::Backend::create("HIP");
    auto a = tensor_of(backend, element::u8, shape_a, vector<uint8_t>{1, 2, 3, 4, 5, 6, 7, 8, 9});
    auto b = tensor_of(backend, element::i8, shape_b, vector<int8_t>{1, 2, 1, 0, 0, 0, -1, -2, -1});
    for (bool f32_bias : {false, true})
    {
        auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
        auto B = make_shared<op::v0::Parameter>(element::i8, shape_b);
        auto Bias = make_shared<op::v0::Parameter>(f32_bias ? element::f32 : element::i32, Shape{1});
        auto CV = builder::QuantizedConvolutionBiasBuilder(A, B, Bias, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1},
                                                           Strides{1, 1}, scalar(0.0f), scalar(255.0f), scalar(-127.0f), scalar(127.0f),
                                                           scalar(20.0f), scalar(-24.0f), true);
        auto f = make_shared<Function>(OutputVector{CV}, ParameterVector{A, B, Bias});
        constant_fold(f);
        auto c = f32_bias ? tensor_of(backend, element::f32, Shape{1}, vector<float>{5}) : tensor_of(backend, element::i32, Shape{1}, vector<int32_t>{5});
        auto result = backend->create_tensor(element::u8, shape_r);
        backend->compile(f)->call_with_validate({result}, {a, b, c});
        EXPECT_VEC_EQ((vector<uint8_t>{0, 0, 0, 0, 0, 0, 191, 255, 234}), read_vector<uint8_t>(result));
    }
}

GPU_TEST(builder, scaled_QC_with_bias_add_and_relu)
{
    Shape shape_a{1, 1, 3, 4}, shape_b{1, 1, 3, 3}, shape_r{1, 1, 3, 4};
    auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto B = make_shared<op::v0::Parameter>(element::i8, shape_b);
    auto Add = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto Bias = make_shared<op::v0::Parameter>(element::i32, Shape{1});
    auto CV = builder::QuantizedConvolutionBiasAddBuilder(A, B, Bias, Add, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1},
                                                          Strides{1, 1}, scalar(0.0f), scalar(255.0f), scalar(-127.0f), scalar(127.0f),
                                                          scalar(22.0f), scalar(90.0f), scalar(22.0f), scalar(180.0f), true);
    auto f = make_shared<Function>(OutputVector{CV}, ParameterVector{A, B, Bias, Add});
    constant_fold(f);
    auto backend = runtime::Backend::create("HIP");
    auto a = tensor_of(backend, element::u8, shape_a, vector<uint8_t>{1, 2, 3, 4, 5, 6, 7, 0, 1, 2, 3, 4});
    auto b = tensor_of(backend, element::i8, shape_b, vector<int8_t>{1, 2, 3, 4, 5, 0, 0, 1, 2});
    auto c = tensor_of(backend, element::i32, Shape{1}, vector<int32_t>{5});
    auto d = tensor_of(backend, element::u8, shape_a, vector<uint8_t>{1, 2, 3, 4, 5, 6, 7, 0, 1, 2, 3, 4});
    auto result = backend->create_tensor(element::u8, shape_r);
    backend->compile(f)->call_with_validate({result}, {a, b, c, d});
    EXPECT_VEC_EQ((vector<uint8_t>{78, 114, 105, 113, 132, 230, 255, 136, 110, 166, 142, 133}), read_vector<uint8_t>(result));
}

GPU_TEST(builder, scaled_QC_with_bias_signed_add_and_relu)
{
    Shape shape_a{1, 1, 3, 4}, shape_b{1, 1, 3, 3}, shape_r{1, 1, 3, 4};
    auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto B = make_shared<op::v0::Parameter>(element::i8, shape_b);
    auto Add = make_shared<op::v0::Parameter>(element::i8, shape_a);
    auto Bias = make_shared<op::v0::Parameter>(element::i32, Shape{1});
    auto CV = builder::QuantizedConvolutionBiasSignedAddBuilder(A, B, Bias, Add, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1},
                                                                CoordinateDiff{1, 1}, Strides{1, 1}, scalar(0.0f), scalar(255.0f), scalar(-127.0f),
                                                                scalar(127.0f), scalar(22.0f), scalar(90.0f), scalar(22.0f), scalar(90.0f), true);
    auto f = make_shared<Function>(OutputVector{CV}, ParameterVector{A, B, Bias, Add});
    constant_fold(f);
    auto backend = runtime::Backend::create("HIP");
    auto a = tensor_of(backend, element::u8, shape_a, vector<uint8_t>{1, 2, 3, 4, 5, 6, 7, 0, 1, 2, 3, 4});
    auto b = tensor_of(backend, element::i8, shape_b, vector<int8_t>{1, 2, 3, 4, 5, 0, 0, 1, 2});
    auto c = tensor_of(backend, element::i32, Shape{1}, vector<int32_t>{5});
    auto d = tensor_of(backend, element::i8, shape_a, vector<int8_t>{-1, -2, -3, -4, -5, -6, -10, 0, 1, 2, 3, 4});
    auto result = backend->create_tensor(element::u8, shape_r);
    backend->compile(f)->call_with_validate({result}, {a, b, c, d});
    EXPECT_VEC_EQ((vector<uint8_t>{74, 106, 93, 97, 112, 127, 127, 127, 110, 127, 127, 127}), read_vector<uint8_t>(result));
}

GPU_TEST(builder, scaled_Q_and_DQ)
{
    auto backend = runtime::Backend::create("HIP");
    auto call_SQ = [&](element::Type type, Shape in_shape, vector<float> in, float min, float max) {
        auto A = make_shared<op::v0::Parameter>(element::f32, in_shape);
        auto B = make_shared<op::v0::Parameter>(element::f32, Shape{});
        auto C = make_shared<op::v0::Parameter>(element::f32, Shape{});
        auto QT = builder::QuantizeBuilder(A, B, C, type, AxisSet{}, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
        auto f = make_shared<Function>(OutputVector{QT}, ParameterVector{A, B, C});
        auto a = tensor_of(backend, element::f32, in_shape, in);
        auto b = tensor_of(backend, element::f32, Shape{}, vector<float>{min});
        auto c = tensor_of(backend, element::f32, Shape{}, vector<float>{max});
        auto result = backend->create_tensor(type, in_shape);
        backend->compile(f)->call_with_validate({result}, {a, b, c});
        return result;
    };
    EXPECT_VEC_EQ((vector<uint8_t>{0, 0, 1, 1, 2, 64, 127, 255}),
                  read_vector<uint8_t>(call_SQ(element::u8, Shape{8}, {-255.0, 0.0, 1.0, 1.25, 1.75, 64.0, 127.0, 500.0}, -255.0f, 127.0f)));
    EXPECT_VEC_EQ((vector<uint8_t>{0, 0, 6, 30, 45, 255, 192, 255}),
                  read_vector<uint8_t>(call_SQ(element::u8, Shape{8}, {-85.0, 0.0, 2.0, 10.0, 15.0, 127.0, 64.0, 500.0}, -85.0f, 15.0f)));
    EXPECT_VEC_EQ((vector<uint8_t>{35, 151, 154, 219}), read_vector<uint8_t>(call_SQ(element::u8, Shape{2, 2}, {0.1392, 0.5928, 0.6027, 0.8579}, 0.0f, 1.0f)));
    EXPECT_VEC_EQ((vector<int8_t>{-86, -90, -127, 10, -5, -19, -35, -20}),
                  read_vector<int8_t>(call_SQ(element::i8, Shape{2, 4},
                                              {-1.3990955, -1.468798, -2.0760186, 0.17088544, -0.0829789, -0.3173087, -0.5645172, -0.3188769},
                                              -2.0760186f, 0.17088544f)));
    EXPECT_VEC_EQ((vector<int8_t>{-127, 0, 1, 3, 5, 64, 127, 127}),
                  read_vector<int8_t>(call_SQ(element::i8, Shape{8}, {-127.0, 0.0, 1.0, 3.0, 5.0, 64.0, 127.0, 500.0}, -127.0f, 127.0f)));

    // DequantizeBuilder with constant ranges, folded
    {
        auto A = make_shared<op::v0::Parameter>(element::i8, Shape{1});
        auto r = builder::DequantizeBuilder(A, scalar(-1.0f), scalar(300.0f), element::f32, AxisSet{});
        auto f = make_shared<Function>(r, ParameterVector{A});
        constant_fold(f);
        auto a = tensor_of(backend, element::i8, Shape{1}, vector<int8_t>{42});
        auto result = backend->create_tensor(element::f32, Shape{1});
        backend->compile(f)->call_with_validate({result}, {a});
        EXPECT_VEC_EQ((vector<float>{99.212601f}), read_vector<float>(result));
    }
    // ... and with ranges fed at call time
    {
        auto A = make_shared<op::v0::Parameter>(element::u8, Shape{2, 2});
        auto B = make_shared<op::v0::Parameter>(element::f32, Shape{});
        auto C = make_shared<op::v0::Parameter>(element::f32, Shape{});
        auto DQT = builder::DequantizeBuilder(A, B, C, element::f32, AxisSet{});
        auto f = make_shared<Function>(OutputVector{DQT}, ParameterVector{A, B, C});
        auto a = tensor_of(backend, element::u8, Shape{2, 2}, vector<uint8_t>{35, 151, 154, 219});
        auto b = tensor_of(backend, element::f32, Shape{}, vector<float>{0.0f});
        auto c = tensor_of(backend, element::f32, Shape{}, vector<float>{1.0f});
        auto result = backend->create_tensor(element::f32, Shape{2, 2});
        backend->compile(f)->call_with_validate({result}, {a, b, c});
        EXPECT_VEC_EQ((vector<float>{0.13725491f, 0.59215689f, 0.60392159f, 0.8588236f}), read_vector<float>(result));
    }
}

GPU_TEST(builder, dynamic_scaled_QD_with_bias)
{
    Shape shape_a{4, 3}, shape_b{3, 3}, shape_c{3}, shape_r{4, 3};
    vector<uint8_t> a_data = {209, 122, 39, 11, 33, 243, 250, 216, 159, 18, 181, 187};
    vector<int8_t> b_data = {11, 15, 80, 50, -6, -3, -6, 78, 113};
    vector<int32_t> c_data = {192, 49, 23};
    auto make_function = [&](bool requantize, bool with_relu) {
        auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
        auto B = make_shared<op::v0::Parameter>(element::i8, shape_b);
        auto Bias = make_shared<op::v0::Parameter>(element::i32, shape_c);
        ParameterVector r;
        for (int i = 0; i < 6; ++i)
            r.push_back(make_shared<op::v0::Parameter>(element::f32, Shape{1}));
        auto CV = builder::QuantizedDotBiasBuilder(A, B, Bias, r[0], r[1], r[2], r[3], r[4], r[5], requantize, with_relu);
        ParameterVector params{A, B, Bias};
        params.insert(params.end(), r.begin(), r.end());
        return make_shared<Function>(OutputVector{CV}, params);
    };
    auto backend = runtime::Backend::create("HIP");
    vector<shared_ptr<runtime::Tensor>> in{tensor_of(backend, element::u8, shape_a, a_data), tensor_of(backend, element::i8, shape_b, b_data),
                                           tensor_of(backend, element::i32, shape_c, c_data)};
    for (float v : {-127.0f, 127.0f, 0.1f, 0.9f, 37.618633f, 2.236754f})
        in.push_back(tensor_of(backend, element::f32, Shape{1}, vector<float>{v}));

    auto r0 = backend->create_tensor(element::f32, shape_r);
    backend->compile(make_function(false, false))->call_with_validate({r0}, in);
    EXPECT_VEC_EQ((vector<float>{26.262351989746094f, 34.05882263183594f, 44.79529571533203f, 71.46353149414062f, -1.1576470136642456f,
                                 105.84706115722656f, 66.71294403076172f, 38.03293991088867f, 117.66352844238281f, 63.75882339477539f,
                                 -2.463529348373413f, 124.10823822021484f}),
                  read_vector<float>(r0));
    auto r1 = backend->create_tensor(element::f32, shape_r);
    backend->compile(make_function(false, true))->call_with_validate({r1}, in);
    EXPECT_VEC_EQ((vector<float>{26.262351989746094f, 34.05882263183594f, 44.79529571533203f, 71.46353149414062f, -0.0f, 105.84706115722656f,
                                 66.71294403076172f, 38.03293991088867f, 117.66352844238281f, 63.75882339477539f, -0.0f, 124.10823822021484f}),
                  read_vector<float>(r1));
    auto r2 = backend->create_tensor(element::i8, shape_r);
    backend->compile(make_function(true, false))->call_with_validate({r2}, in);
    EXPECT_VEC_EQ((vector<int8_t>{89, 115, 127, 127, -4, 127, 127, 127, 127, 127, -8, 127}), read_vector<int8_t>(r2));
    auto r3 = backend->create_tensor(element::u8, shape_r);
    backend->compile(make_function(true, true))->call_with_validate({r3}, in);
    EXPECT_VEC_EQ((vector<uint8_t>{178, 231, 255, 255, 0, 255, 255, 255, 255, 255, 0, 255}), read_vector<uint8_t>(r3));
}
