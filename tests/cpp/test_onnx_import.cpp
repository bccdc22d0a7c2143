// ONNX model ingress: the reader against the models of tests/golden/onnx (written by
// tests/golden/make_onnx_models.py as text and as binary protobuf; the graphs restate those of the
// reference's importer tests), the graphs it builds, and those graphs on backend "HIP" against the
// expected vectors of test/onnx/onnx_import_quant.in.cpp of the nGraph tree (cited at each case).
#include <fstream>
#include <sstream>
#include <unistd.h>

#include "ngraph/frontend/onnx_import/onnx.hpp"
#include "ngraph/serializer.hpp"
#include "test_util.hpp"

using namespace std;
using namespace ngraph;

namespace
{
    string golden(const string& file)
    {
        // the test binary lives in ngraph_amd/host/, the fixtures in tests/golden/
        char buf[4096];
        ssize_t n = ::readlink("/proc/self/exe", buf, sizeof buf - 1);
        string exe = n > 0 ? string(buf, static_cast<size_t>(n)) : string();
        string dir = exe.substr(0, exe.find_last_of('/'));
        return dir + "/../../tests/golden/" + file;
    }

    const char* const kFormats[] = {".prototxt", ".onnx"};

    shared_ptr<Function> load(const string& model, const string& format) { return onnx_import::import_onnx_model(golden("onnx/" + model + format)); }

    string what_of(const function<void()>& fn)
    {
        try
        {
            fn();
        }
        catch (const exception& e)
        {
            return e.what();
        }
        return "";
    }

    template <typename T>
    shared_ptr<T> only(const shared_ptr<Function>& f)
    {
        shared_ptr<T> found;
        for (const auto& n : f->get_ordered_ops())
            if (auto t = as_type_ptr<T>(n))
            {
                EXPECT_TRUE(!found);
                found = t;
            }
        EXPECT_TRUE(found != nullptr);
        return found;
    }

    vector<uint8_t> file_bytes(const string& path)
    {
        ifstream in(path, ios::binary);
        if (!in)
            throw runtime_error("cannot open " + path);
        stringstream ss;
        ss << in.rdbuf();
        const string s = ss.str();
        return vector<uint8_t>(s.begin(), s.end());
    }

    // one input of a call: element type + bytes
    struct In
    {
        element::Type type;
        vector<uint8_t> bytes;
    };
    template <typename T>
    In in(const vector<T>& v)
    {
        In i{element::from<T>(), vector<uint8_t>(v.size() * sizeof(T))};
        memcpy(i.bytes.data(), v.data(), i.bytes.size());
        return i;
    }

    // runs the model (both file formats) on "HIP" with the given inputs and checks its one output
    template <typename T>
    void expect_output(const string& model, const vector<In>& inputs, const Shape& shape, const vector<T>& expected)
    {
        auto backend = runtime::Backend::create("HIP");
        for (const char* format : kFormats)
        {
            auto f = load(model, format);
            EXPECT_EQ(f->get_parameters().size(), inputs.size());
            EXPECT_EQ(f->get_output_shape(0), shape);
            EXPECT_EQ(f->get_output_element_type(0), element::from<T>());
            vector<shared_ptr<runtime::Tensor>> args;
            for (size_t i = 0; i < inputs.size(); ++i)
            {
                const auto& p = f->get_parameters().at(i);
                EXPECT_EQ(p->get_output_element_type(0), inputs[i].type);
                EXPECT_EQ(shape_size(p->get_output_shape(0)) * inputs[i].type.size(), inputs[i].bytes.size());
                auto t = backend->create_tensor(p->get_output_element_type(0), p->get_output_shape(0));
                t->write(inputs[i].bytes.data(), inputs[i].bytes.size());
                args.push_back(t);
            }
            auto result = backend->create_tensor(element::from<T>(), shape);
            backend->compile(f)->call_with_validate({result}, args);
            EXPECT_VEC_EQ(expected, read_vector<T>(result));
        }
    }
}

// ---------------------------------------------------------------------------------- reader, CPU
CPU_TEST(onnx_import, quantize_linear_graphs)
{
    for (const char* format : kFormats)
    {
        // the zero point comes from an initializer: a Constant, not a Parameter
        auto f = load("quantize_linear", format);
        EXPECT_EQ(f->get_name(), string("test_graph"));
        EXPECT_EQ(f->get_parameters().size(), size_t(2));
        EXPECT_EQ(f->get_parameters()[0]->get_friendly_name(), string("x"));
        EXPECT_EQ(f->get_parameters()[1]->get_friendly_name(), string("y_scale"));
        auto q = only<op::v0::Quantize>(f);
        EXPECT_TRUE(q->get_round_mode() == op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
        EXPECT_TRUE(q->get_axes().empty());
        EXPECT_EQ(q->get_output_element_type(0), element::u8);
        EXPECT_EQ(q->get_output_shape(0), (Shape{2, 2}));
        auto zp = as_type_ptr<op::v0::Constant>(q->get_argument(2));
        EXPECT_TRUE(zp != nullptr);
        EXPECT_EQ(zp->get_output_element_type(0), element::u8);
        EXPECT_VEC_EQ((vector<uint8_t>{0}), zp->get_vector<uint8_t>());
        EXPECT_EQ(f->get_output_op(0)->get_friendly_name(), string("y"));

        // axis given: that axis; negative: counted from the end
        EXPECT_EQ(only<op::v0::Quantize>(load("quantize_linear_axis_zero", format))->get_axes(), (AxisSet{0}));
        EXPECT_EQ(only<op::v0::Quantize>(load("quantize_linear_axis_negative", format))->get_axes(), (AxisSet{0}));
        EXPECT_EQ(only<op::v0::Dequantize>(load("dequantize_linear_axis1_4d", format))->get_axes(), (AxisSet{1}));
        EXPECT_EQ(only<op::v0::Dequantize>(load("dequantize_linear_axis_negative", format))->get_axes(), (AxisSet{0}));
        EXPECT_TRUE(only<op::v0::Dequantize>(load("dequantize_linear_u8", format))->get_axes().empty());
    }
}

CPU_TEST(onnx_import, convolution_and_matmul_graphs)
{
    for (const char* format : kFormats)
    {
        // every side input an initializer; the filter's initializer is i8 although the input list says u8
        auto f = load("qlinear_conv_initializers", format);
        EXPECT_EQ(f->get_parameters().size(), size_t(1));
        auto cv = only<op::v0::QuantizedConvolution>(f);
        EXPECT_EQ(cv->get_argument(1)->get_output_element_type(0), element::i8);
        EXPECT_VEC_EQ((vector<int8_t>{1, 0, 2, 1, 0, 2, 1, 0, 2}), as_type_ptr<op::v0::Constant>(cv->get_argument(1))->get_vector<int8_t>());
        EXPECT_EQ(cv->get_output_element_type(0), element::i8);
        EXPECT_EQ(cv->get_output_shape(0), (Shape{1, 1, 9, 9}));
        EXPECT_EQ(cv->get_padding_below(), (CoordinateDiff{1, 1}));
        EXPECT_EQ(cv->get_padding_above(), (CoordinateDiff{1, 1}));
        EXPECT_EQ(cv->get_window_movement_strides(), (Strides{1, 1}));
        EXPECT_VEC_EQ((vector<float>{16.0f}), as_type_ptr<op::v0::Constant>(cv->get_argument(6))->get_vector<float>());

        auto c3 = only<op::v0::QuantizedConvolution>(load("qlinear_conv_3d", format));
        EXPECT_EQ(c3->get_window_movement_strides(), (Strides{2, 2, 2}));
        EXPECT_EQ(c3->get_window_dilation_strides(), (Strides{1, 1, 1}));
        EXPECT_EQ(c3->get_data_dilation_strides(), (Strides{1, 1, 1}));
        EXPECT_EQ(c3->get_padding_below(), (CoordinateDiff{2, 2, 2}));
        EXPECT_EQ(c3->get_padding_above(), (CoordinateDiff{2, 2, 2}));
        EXPECT_EQ(c3->get_output_element_type(0), element::u8);
        EXPECT_EQ(c3->get_output_shape(0), (Shape{1, 1, 4, 4, 4}));

        // ConvInteger: unit scales, i32 output, zero points of the operands' types where none is given
        auto ci = only<op::v0::QuantizedConvolution>(load("conv_integer_no_zero_point", format));
        EXPECT_EQ(ci->get_output_element_type(0), element::i32);
        EXPECT_EQ(ci->get_argument(3)->get_output_element_type(0), element::u8);
        EXPECT_EQ(ci->get_argument(7)->get_output_element_type(0), element::i32);
        EXPECT_VEC_EQ((vector<float>{1.0f}), as_type_ptr<op::v0::Constant>(ci->get_argument(2))->get_vector<float>());
        auto cp = only<op::v0::QuantizedConvolution>(load("conv_integer_pads", format));
        EXPECT_EQ(cp->get_padding_below(), (CoordinateDiff{1, 1}));
        EXPECT_EQ(cp->get_output_shape(0), (Shape{1, 1, 4, 4}));
        // automatic padding (validation_util.cpp:604-627): one row and column more, above or below
        auto up = only<op::v0::QuantizedConvolution>(load("conv_integer_same_upper", format));
        EXPECT_EQ(up->get_padding_below(), (CoordinateDiff{0, 0}));
        EXPECT_EQ(up->get_padding_above(), (CoordinateDiff{1, 1}));
        auto lo = only<op::v0::QuantizedConvolution>(load("conv_integer_same_lower", format));
        EXPECT_EQ(lo->get_padding_below(), (CoordinateDiff{1, 1}));
        EXPECT_EQ(lo->get_padding_above(), (CoordinateDiff{0, 0}));

        auto qd = only<op::v0::QuantizedDot>(load("qlinear_matmul", format));
        EXPECT_EQ(qd->get_reduction_axes_count(), size_t(1));
        EXPECT_EQ(qd->get_output_element_type(0), element::u8);
        EXPECT_EQ(qd->get_output_shape(0), (Shape{2, 3}));
        auto mi = only<op::v0::QuantizedDot>(load("matmul_integer", format));
        EXPECT_EQ(mi->get_output_element_type(0), element::i32);
        EXPECT_EQ(mi->get_output_shape(0), (Shape{4, 2}));
        EXPECT_TRUE(mi->get_argument(3)->is_parameter() && mi->get_argument(5)->is_parameter());
        auto mn = only<op::v0::QuantizedDot>(load("matmul_integer_no_zero_point", format));
        EXPECT_TRUE(mn->get_argument(3)->is_constant() && mn->get_argument(5)->is_constant());

        // Constant nodes and glue
        auto chain = load("dequantize_relu_quantize", format);
        EXPECT_EQ(chain->get_parameters().size(), size_t(1));
        EXPECT_EQ(count_ops_of_type<op::v0::Constant>(chain), size_t(2));
        EXPECT_EQ(count_ops_of_type<op::v0::Relu>(chain), size_t(1));
        auto dq = only<op::v0::Dequantize>(chain);
        EXPECT_VEC_EQ((vector<float>{0.5f}), as_type_ptr<op::v0::Constant>(dq->get_argument(1))->get_vector<float>());
        EXPECT_EQ(dq->get_friendly_name(), string("real"));
    }
}

CPU_TEST(onnx_import, text_and_binary_files_give_the_same_graph)
{
    // serialized, the two graphs differ in nothing but the process-wide instance numbers of their
    // node names: compare op by op instead
    for (const string model : {"qlinear_conv_3d", "dequantize_relu_quantize", "matmul_integer", "qlinear_conv_initializers"})
    {
        auto a = load(model, ".prototxt")->get_ordered_ops();
        auto b = load(model, ".onnx")->get_ordered_ops();
        EXPECT_EQ(a.size(), b.size());
        for (size_t i = 0; i < a.size() && i < b.size(); ++i)
        {
            EXPECT_EQ(string(a[i]->get_type_info().name), string(b[i]->get_type_info().name));
            EXPECT_EQ(a[i]->get_friendly_name().substr(0, 1), b[i]->get_friendly_name().substr(0, 1));
            EXPECT_EQ(a[i]->get_output_size(), b[i]->get_output_size());
            for (size_t o = 0; o < a[i]->get_output_size(); ++o)
            {
                EXPECT_EQ(a[i]->get_output_shape(o), b[i]->get_output_shape(o));
                EXPECT_EQ(a[i]->get_output_element_type(o), b[i]->get_output_element_type(o));
            }
            if (auto ca = as_type_ptr<op::v0::Constant>(a[i]))
                EXPECT_VEC_EQ(ca->get_values_as_double(), as_type_ptr<op::v0::Constant>(b[i])->get_values_as_double());
        }
    }
    // and a model survives this library's serializer
    auto f = load("qlinear_conv_3d", ".onnx");
    auto g = deserialize(serialize(f, 2));
    EXPECT_EQ(only<op::v0::QuantizedConvolution>(g)->get_padding_above(), (CoordinateDiff{2, 2, 2}));
}

CPU_TEST(onnx_import, errors_and_operator_queries)
{
    EXPECT_TRUE(what_of([] { onnx_import::import_onnx_model(golden("onnx/no_such_model.onnx")); }).find("Failure opening file") != string::npos);
    {
        stringstream garbage("this is neither kind of protobuf {{{");
        EXPECT_TRUE(what_of([&] { onnx_import::import_onnx_model(garbage); }).find("Failure parsing data from the provided input stream") != string::npos);
        stringstream empty("");
        EXPECT_TRUE(what_of([&] { onnx_import::import_onnx_model(empty); }).find("Failure parsing data") != string::npos);
        // a binary file cut short falls through both readers
        const auto bytes = file_bytes(golden("onnx/qlinear_matmul.onnx"));
        stringstream cut(string(bytes.begin(), bytes.begin() + static_cast<ptrdiff_t>(bytes.size() / 2)));
        EXPECT_TRUE(!what_of([&] { onnx_import::import_onnx_model(cut); }).empty());
    }
    for (const char* format : kFormats)
    {
        EXPECT_TRUE(what_of([&] { load("unsupported_operator", format); }).find("unsupported operator Softplus (opset 10)") != string::npos);
        // stack axes are broadcast numpy-style (builder/autobroadcast.cpp:285-318); stacks of 2 and of 3 matrices do not fit
        EXPECT_TRUE(what_of([&] { load("matmul_integer_stacks_clash", format); }).find("cannot be broadcast") != string::npos);
    }
    EXPECT_TRUE(onnx_import::is_operator_supported("QLinearConv", 10, "ai.onnx"));
    EXPECT_TRUE(onnx_import::is_operator_supported("QuantizeLinear", 10, ""));
    EXPECT_TRUE(!onnx_import::is_operator_supported("QLinearConv", 10, "com.example"));
    EXPECT_TRUE(!onnx_import::is_operator_supported("Softplus", 10, "ai.onnx"));
    const auto ops = onnx_import::get_supported_operators(10, "ai.onnx");
    for (const char* op : {"QuantizeLinear", "DequantizeLinear", "QLinearConv", "QLinearMatMul", "ConvInteger", "MatMulInteger"})
        EXPECT_TRUE(ops.count(op) == 1);
}

CPU_TEST(onnx_import, qlinear_conv_with_bias_builds_the_reference_subgraph)
{
    // builder/quantization/quantized_linear_convolution.cpp:38-77: QuantizedConvolutionBias whose scale
    // input is (x_scale * w_scale) / y_scale as graph nodes; an int32 bias goes in as it is
    for (const char* format : kFormats)
    {
        auto f = load("qlinear_conv_bias", format);
        EXPECT_EQ(f->get_parameters().size(), size_t(1));
        auto cb = only<op::v0::QuantizedConvolutionBias>(f);
        EXPECT_TRUE(!cb->with_relu());
        EXPECT_EQ(cb->get_output_element_type(0), element::i8);
        EXPECT_EQ(cb->get_argument(2)->get_output_element_type(0), element::i32);
        EXPECT_TRUE(cb->get_argument(2)->is_constant());
        auto div = as_type_ptr<op::v1::Divide>(cb->get_argument(3));
        EXPECT_TRUE(div != nullptr);
        EXPECT_TRUE(as_type_ptr<op::v1::Multiply>(div->get_argument(0)) != nullptr);
        EXPECT_VEC_EQ((vector<float>{0.125f}), as_type_ptr<op::v0::Constant>(div->get_argument(1))->get_vector<float>());
    }
}

CPU_TEST(onnx_import, damaged_files_are_refused_not_crashed_on)
{
    // every prefix of a binary and of a text model, and both with single bytes flipped: the reader
    // either builds a graph or throws -- no reads past the end, no unbounded recursion or allocation
    size_t built = 0, refused = 0;
    auto attempt = [&](const string& bytes) {
        stringstream ss(bytes);
        try
        {
            onnx_import::import_onnx_model(ss);
            ++built;
        }
        catch (const exception&)
        {
            ++refused;
        }
    };
    for (const char* format : kFormats)
    {
        const auto raw = file_bytes(golden(string("onnx/qlinear_conv_initializers") + format));
        const string whole(raw.begin(), raw.end());
        for (size_t n = 0; n < whole.size(); n += (whole.size() > 2000 ? 7 : 1))
            attempt(whole.substr(0, n));
        uint32_t state = 12345;
        for (int round = 0; round < 3000; ++round)
        {
            state = state * 1664525u + 1013904223u;
            string damaged = whole;
            damaged[(state >> 8) % damaged.size()] = static_cast<char>(state >> 24);
            attempt(damaged);
        }
    }
    EXPECT_TRUE(refused > 100);
    EXPECT_TRUE(built > 0); // (a flipped byte inside a name or a number still gives a model)
}

CPU_TEST(onnx_import, stacks_of_matrices_and_grouped_convolutions)
{
    for (const char* format : kFormats)
    {
        // builder/matmul_factory.cpp:88-150: a QuantizedDot a matrix of the (collapsed) stack between Slice
        // and Concat, the stack axes restored by a Reshape
        auto f = load("matmul_integer_4d", format);
        EXPECT_EQ(f->get_output_shape(0), (Shape{1, 2, 3, 3}));
        EXPECT_EQ(f->get_output_element_type(0), element::i32);
        EXPECT_EQ(count_ops_of_type<op::v0::QuantizedDot>(f), size_t(2));
        EXPECT_EQ(count_ops_of_type<op::v0::Slice>(f), size_t(4));
        EXPECT_EQ(count_ops_of_type<op::v0::Concat>(f), size_t(1));
        auto g = load("qlinear_matmul_3d", format);
        EXPECT_EQ(g->get_output_shape(0), (Shape{2, 2, 3}));
        EXPECT_EQ(count_ops_of_type<op::v0::QuantizedDot>(g), size_t(2));
        // quant_conv.cpp:80-138: a convolution a group on channel slices, concatenated on the channel axis
        auto h = load("qlinear_conv_groups", format);
        EXPECT_EQ(h->get_output_shape(0), (Shape{1, 2, 2, 2}));
        EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolution>(h), size_t(2));
        EXPECT_EQ(count_ops_of_type<op::v0::Slice>(h), size_t(4));
        EXPECT_EQ(only<op::v0::Concat>(h)->get_concatenation_axis(), int64_t(1));
    }
}

// ---------------------------------------------------------------------------------- on the device
// test/onnx/onnx_import_quant.in.cpp:44-108
GPU_TEST(onnx_import, quantize_linear_vectors)
{
    expect_output<uint8_t>("quantize_linear", {in<float>({32.25f, 48.34f, 50.f, 83.f}), in<float>({0.5f})}, Shape{2, 2}, {64, 97, 100, 166});
    expect_output<uint8_t>("quantize_linear_zero_point", {in<float>({0.f, 2.f, 3.f, 1000.f, -254.f, -1000.f}), in<float>({2.0f}), in<uint8_t>({128})}, Shape{6}, {128, 129, 130, 255, 1, 0});
    const vector<float> x{0.f, 2.f, 3.f, 1000.f, 0.f, 2.f, 3.f, 1000.f, 0.f, 2.f, 3.f, 1000.f};
    for (const char* model : {"quantize_linear_axis_zero", "quantize_linear_axis_negative"})
        expect_output<uint8_t>(model, {in(x), in<float>({1.f, 2.f, 4.f}), in<uint8_t>({0, 0, 0})}, Shape{3, 4}, {0, 2, 3, 255, 0, 1, 2, 255, 0, 0, 1, 250});
}

// :110-227
GPU_TEST(onnx_import, dequantize_linear_vectors)
{
    expect_output<float>("dequantize_linear_initializers", {in<uint8_t>({19, 210, 21, 10})}, Shape{2, 2}, {76.f, 840.f, 84.f, 40.f});
    expect_output<float>("dequantize_linear_u8", {in<uint8_t>({0, 3, 128, 255}), in<float>({2.0f}), in<uint8_t>({128})}, Shape{4}, {-256.0f, -250.0f, 0.0f, 254.0f});
    expect_output<float>("dequantize_linear_i8", {in<int8_t>({-30, -3, 100, 127}), in<float>({2.0f}), in<int8_t>({-10})}, Shape{4}, {-40.0f, 14.0f, 220.0f, 274.0f});
    for (const char* model : {"dequantize_linear_axis0_u8", "dequantize_linear_axis_negative"})
        expect_output<float>(model,
                             {in<uint8_t>({0, 1, 2, 3, 0, 1, 2, 3, 0, 10, 20, 30}), in<float>({1.0f, 2.0f, 4.0f}), in<uint8_t>({0, 0, 0})},
                             Shape{3, 4},
                             {0.0f, 1.0f, 2.0f, 3.0f, 0.0f, 2.0f, 4.0f, 6.0f, 0.0f, 40.0f, 80.0f, 120.0f});
    expect_output<float>("dequantize_linear_axis1_i8",
                         {in<int8_t>({0, 1, 2, 3, 0, 2, 4, 6, 0, 10, 20, 30}), in<float>({1.0f, 2.0f, 4.0f, 8.0f}), in<int8_t>({0, -10, -20, -30})},
                         Shape{3, 4},
                         {0.0f, 22.0f, 88.0f, 264.0f, 0.0f, 24.0f, 96.0f, 288.0f, 0.0f, 40.0f, 160.0f, 480.0f});
    expect_output<float>("dequantize_linear_axis1_4d",
                         {in<uint8_t>({7, 9, 10, 10, 5, 8, 9, 1, 8, 6, 7, 9, 10, 0, 7, 10, 8, 2, 6, 0, 5, 9, 8, 1, 2, 7, 5, 3, 2, 4, 1, 3, 8, 7, 4, 8, 10, 1, 5, 5, 7, 7, 0, 2, 4, 4, 0, 5}),
                          in<float>({1.0f, 10.0f, 7.0f}),
                          in<uint8_t>({10, 2, 1})},
                         Shape{2, 3, 2, 4},
                         {-3.0f, -1.0f, 0.0f,  0.0f,  -5.0f, -2.0f, -1.0f, -9.0f, 60.0f, 40.0f, 50.0f, 70.0f, 80.0f, -20.0f, 50.0f, 80.0f,
                          49.0f, 7.0f,  35.0f, -7.0f, 28.0f, 56.0f, 49.0f, 0.0f,  -8.0f, -3.0f, -5.0f, -7.0f, -8.0f, -6.0f,  -9.0f, -7.0f,
                          60.0f, 50.0f, 20.0f, 60.0f, 80.0f, -10.0f, 30.0f, 30.0f, 42.0f, 42.0f, -7.0f, 7.0f,  21.0f, 21.0f,  -7.0f, 28.0f});
}

// :229-292
GPU_TEST(onnx_import, qlinear_conv_vectors)
{
    vector<uint8_t> ramp(81);
    for (size_t i = 0; i < ramp.size(); ++i)
        ramp[i] = static_cast<uint8_t>(i + 1);
    // The reference's vector (:239-246) with its two exact ties, 264 / 16 and 552 / 16 at elements 28
    // and 60, rounded away from zero: QuantizedConvolution follows the INTERPRETER kernel's std::round
    // (src/ngraph/runtime/reference/convolution.hpp:255), the vector there holds 16 and 34, the
    // round-half-even of the CPU backend it was recorded on.
    expect_output<int8_t>("qlinear_conv_initializers",
                          {in(ramp)},
                          Shape{1, 1, 9, 9},
                          {2,  3,  3,  3,  4,  4,  4,  5,  2,  4,  6,  7,  8,  8,  9,  9,  10, 3,  8,  11, 12, 13, 13, 14, 14, 15, 5,
                           11, 17, 17, 18, 18, 19, 19, 20, 7,  14, 22, 22, 23, 23, 24, 24, 25, 8,  18, 27, 27, 28, 28, 29, 29, 30, 10,
                           21, 32, 32, 33, 33, 34, 35, 35, 12, 24, 37, 37, 38, 38, 39, 40, 40, 13, 17, 26, 27, 27, 27, 28, 28, 28, 9});
    // the data files of the reference's tests (test/files/onnx/qlinearconv2d, qlinearconv3d): non-zero zero points
    expect_output<uint8_t>("qlinear_conv_2d",
                           {In{element::u8, file_bytes(golden("qlinearconv2d_x.bin"))}, in<float>({0.00369204697199166f}), in<uint8_t>({132}), in<uint8_t>({0}),
                            in<float>({0.00172794575337321f}), in<uint8_t>({255}), in<float>({0.00162681262008846f}), in<uint8_t>({123})},
                           Shape{1, 1, 7, 7},
                           file_bytes(golden("qlinearconv2d_y.bin")));
    expect_output<uint8_t>("qlinear_conv_3d",
                           {In{element::u8, file_bytes(golden("qlinearconv3d_x.bin"))}, in<float>({0.00389225385151803f}), in<uint8_t>({127}), in<uint8_t>({255}),
                            in<float>({0.00128723995294422f}), in<uint8_t>({0}), in<float>({0.0011764180380851f}), in<uint8_t>({128})},
                           Shape{1, 1, 4, 4, 4},
                           file_bytes(golden("qlinearconv3d_y.bin")));
}

// :294-313, :340-456
GPU_TEST(onnx_import, matmul_and_conv_integer_vectors)
{
    expect_output<uint8_t>("qlinear_matmul",
                           {in<uint8_t>({208, 236, 0, 238, 3, 214, 255, 29}), in<float>({0.0066f}), in<uint8_t>({113}), in<uint8_t>({152, 51, 244, 60, 26, 255, 0, 127, 246, 127, 254, 247}),
                            in<float>({0.00705f}), in<uint8_t>({114}), in<float>({0.0107f}), in<uint8_t>({118})},
                           Shape{2, 3},
                           {168, 115, 255, 1, 66, 151});
    expect_output<int32_t>("conv_integer", {in<uint8_t>({2, 3, 4, 5, 6, 7, 8, 9, 10}), in<uint8_t>({1, 1, 1, 1}), in<uint8_t>({1})}, Shape{1, 1, 2, 2}, {12, 16, 24, 28});
    expect_output<int32_t>("conv_integer", {in<uint8_t>({1, 2, 3, 4, 5, 6, 7, 8, 9}), in<uint8_t>({1, 1, 1, 1}), in<uint8_t>({0})}, Shape{1, 1, 2, 2}, {12, 16, 24, 28});
    expect_output<int32_t>("conv_integer_no_zero_point", {in<uint8_t>({1, 2, 3, 4, 5, 6, 7, 8, 9}), in<uint8_t>({1, 1, 1, 1})}, Shape{1, 1, 2, 2}, {12, 16, 24, 28});
    expect_output<int32_t>("conv_integer_pads",
                           {in<uint8_t>({2, 3, 4, 5, 6, 7, 8, 9, 10}), in<uint8_t>({1, 1, 1, 1}), in<uint8_t>({1})},
                           Shape{1, 1, 4, 4},
                           {1, 3, 5, 3, 5, 12, 16, 9, 11, 24, 28, 15, 7, 15, 17, 9});
    const vector<uint8_t> a{11, 7, 3, 10, 6, 2, 9, 5, 1, 8, 4, 0}, b{1, 4, 2, 5, 3, 6};
    expect_output<int32_t>("matmul_integer", {in(a), in(b), in<uint8_t>({12}), in<uint8_t>({0})}, Shape{4, 2}, {-38, -83, -44, -98, -50, -113, -56, -128});
    expect_output<int32_t>("matmul_integer", {in(a), in(b), in<uint8_t>({0}), in<uint8_t>({0})}, Shape{4, 2}, {34, 97, 28, 82, 22, 67, 16, 52});
    expect_output<int32_t>("matmul_integer_no_zero_point", {in(a), in(b)}, Shape{4, 2}, {34, 97, 28, 82, 22, 67, 16, 52});
    expect_output<int32_t>("matmul_integer_scalar", {in<uint8_t>({11}), in<uint8_t>({13}), in<uint8_t>({12}), in<uint8_t>({12})}, Shape{1, 1}, {-1});
}

// :315-338, :458-560: stacks of matrices
GPU_TEST(onnx_import, stacked_matmul_vectors)
{
    expect_output<uint8_t>("qlinear_matmul_3d",
                           {in<uint8_t>({208, 236, 0, 238, 3, 214, 255, 29, 208, 236, 0, 238, 3, 214, 255, 29}), in<float>({0.0066f}), in<uint8_t>({113}),
                            in<uint8_t>({152, 51, 244, 60, 26, 255, 0, 127, 246, 127, 254, 247, 152, 51, 244, 60, 26, 255, 0, 127, 246, 127, 254, 247}), in<float>({0.00705f}), in<uint8_t>({114}),
                            in<float>({0.0107f}), in<uint8_t>({118})},
                           Shape{2, 2, 3},
                           {168, 115, 255, 1, 66, 151, 168, 115, 255, 1, 66, 151});
    vector<uint8_t> ramp(24);
    for (size_t i = 0; i < ramp.size(); ++i)
        ramp[i] = static_cast<uint8_t>(i);
    const vector<int32_t> plain{42, 48, 54, 114, 136, 158, 186, 224, 262, 906, 960, 1014, 1170, 1240, 1310, 1434, 1520, 1606};
    expect_output<int32_t>("matmul_integer_4d", {in(ramp), in(ramp), in<uint8_t>({0}), in<uint8_t>({0})}, Shape{1, 2, 3, 3}, plain);
    expect_output<int32_t>("matmul_integer_4d", {in(ramp), in(ramp), in<uint8_t>({1}), in<uint8_t>({1})}, Shape{1, 2, 3, 3},
                           {22, 24, 26, 78, 96, 114, 134, 168, 202, 790, 840, 890, 1038, 1104, 1170, 1286, 1368, 1450});
    expect_output<int32_t>("matmul_integer_4d_no_zero_point", {in(ramp), in(ramp)}, Shape{1, 2, 3, 3}, plain);
    // (not from the reference's tests) two groups of one channel under 1 x 1 filters 2 and 3
    expect_output<int8_t>("qlinear_conv_groups", {in<uint8_t>({1, 2, 3, 4, 5, 6, 7, 8})}, Shape{1, 2, 2, 2}, {2, 4, 6, 8, 15, 18, 21, 24});
}

// builder/matmul_factory.cpp:88-105 with builder/autobroadcast.cpp:285-318: the stack axes of the two
// operands are broadcast against each other numpy-style before the stack is multiplied matrix by matrix.
// Expected values: the products written out as loops here (numpy.matmul's definition).
namespace
{
    // a [.., M, K] by b [.., K, N] with the stack axes of both already repeated to `stack` (row-major);
    // la / lb give, for every matrix of the result, which matrix of a / b it multiplies
    vector<int32_t> stacked_product(const vector<uint8_t>& a, const vector<uint8_t>& b, const vector<size_t>& la, const vector<size_t>& lb, size_t M, size_t K, size_t N, int azp, int bzp)
    {
        vector<int32_t> y(la.size() * M * N);
        for (size_t g = 0; g < la.size(); ++g)
            for (size_t m = 0; m < M; ++m)
                for (size_t n = 0; n < N; ++n)
                {
                    int32_t acc = 0;
                    for (size_t k = 0; k < K; ++k)
                        acc += (static_cast<int>(a[(la[g] * M + m) * K + k]) - azp) * (static_cast<int>(b[(lb[g] * K + k) * N + n]) - bzp);
                    y[(g * M + m) * N + n] = acc;
                }
        return y;
    }
}

CPU_TEST(onnx_import, stack_axes_are_broadcast)
{
    for (const char* format : kFormats)
    {
        // [2, 3, 4] x [1, 4, 3]: the right operand loses its axis of length 1 (Reshape) and is repeated (Broadcast)
        auto f = load("matmul_integer_broadcast_3d", format);
        EXPECT_EQ(f->get_output_shape(0), (Shape{2, 3, 3}));
        EXPECT_EQ(count_ops_of_type<op::v0::Broadcast>(f), size_t(1));
        EXPECT_EQ(count_ops_of_type<op::v0::QuantizedDot>(f), size_t(2));
        // [2, 1, 3, 4] x [1, 3, 4, 2]: both repeated to a [2, 3] stack, six products
        auto g = load("matmul_integer_broadcast_4d", format);
        EXPECT_EQ(g->get_output_shape(0), (Shape{2, 3, 3, 2}));
        EXPECT_EQ(count_ops_of_type<op::v0::Broadcast>(g), size_t(2));
        EXPECT_EQ(count_ops_of_type<op::v0::QuantizedDot>(g), size_t(6));
        // [3, 4] x [2, 4, 3]: the matrix is repeated for every matrix of the stack
        auto h = load("matmul_integer_matrix_by_stack", format);
        EXPECT_EQ(h->get_output_shape(0), (Shape{2, 3, 3}));
        EXPECT_EQ(count_ops_of_type<op::v0::Broadcast>(h), size_t(1));
    }
}

GPU_TEST(onnx_import, stack_axes_are_broadcast_vectors)
{
    auto ramp = [](size_t n, int step, int start) {
        vector<uint8_t> v(n);
        for (size_t i = 0; i < n; ++i)
            v[i] = static_cast<uint8_t>((start + static_cast<int>(i) * step) & 0xFF);
        return v;
    };
    {
        const auto a = ramp(24, 7, 3), b = ramp(12, 11, 5);
        expect_output<int32_t>("matmul_integer_broadcast_3d", {in(a), in(b), in<uint8_t>({2}), in<uint8_t>({9})}, Shape{2, 3, 3}, stacked_product(a, b, {0, 1}, {0, 0}, 3, 4, 3, 2, 9));
    }
    {
        // result stack [2, 3]: matrix (i, j) is a[i] x b[j]
        const auto a = ramp(24, 13, 1), b = ramp(24, 5, 200);
        expect_output<int32_t>("matmul_integer_broadcast_4d", {in(a), in(b), in<uint8_t>({100}), in<uint8_t>({0})}, Shape{2, 3, 3, 2},
                               stacked_product(a, b, {0, 0, 0, 1, 1, 1}, {0, 1, 2, 0, 1, 2}, 3, 4, 2, 100, 0));
    }
    {
        const auto a = ramp(12, 17, 9), b = ramp(24, 3, 50);
        expect_output<int32_t>("matmul_integer_matrix_by_stack", {in(a), in(b), in<uint8_t>({0}), in<uint8_t>({60})}, Shape{2, 3, 3}, stacked_product(a, b, {0, 0}, {0, 1}, 3, 4, 3, 0, 60));
    }
}

// not from the reference's tests: window sums worked by hand (a 4 x 4 ramp 0..15 under a 3 x 3 window
// of ones at stride 2, the missing row and column above or below the data), and a chain through glue
GPU_TEST(onnx_import, automatic_padding_and_glue_chain)
{
    vector<uint8_t> ramp(16);
    for (size_t i = 0; i < ramp.size(); ++i)
        ramp[i] = static_cast<uint8_t>(i);
    const vector<uint8_t> ones(9, 1);
    expect_output<int32_t>("conv_integer_same_upper", {in(ramp), in(ones)}, Shape{1, 1, 2, 2}, {45, 39, 66, 50});
    expect_output<int32_t>("conv_integer_same_lower", {in(ramp), in(ones)}, Shape{1, 1, 2, 2}, {10, 24, 51, 90});
    // Dequantize (scale 0.5) -> Relu -> Quantize (scale 0.5): negatives to zero, everything else unchanged
    expect_output<int8_t>("dequantize_relu_quantize", {in<int8_t>({-4, -1, 0, 1, 5, 127})}, Shape{2, 3}, {0, 0, 0, 1, 5, 127});
    // QLinearConv with an int32 bias: 1 x 1 filter 2, requantization scale 1: 2 x + 10, saturated to i8
    expect_output<int8_t>("qlinear_conv_bias", {in<uint8_t>({1, 2, 3, 100})}, Shape{1, 1, 2, 2}, {12, 14, 16, 127});
}
