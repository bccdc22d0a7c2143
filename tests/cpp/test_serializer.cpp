// JSON model ingress: the reader against hand-restated nGraph-format files (tests/golden/serialized,
// written by tests/golden/make_serialized_graphs.py from the graphs of the reference's backend
// tests), the writer through round trips, and the loaded graphs on backend "HIP" against the
// expected vectors of those reference tests (test/backend/quantized_convolution.in.cpp,
// quantized_dot.in.cpp:31-115, quantize_dequantize.in.cpp:31-108).  Pattern of the reference's
// test/serialize.cpp: serialize -> deserialize -> run -> compare.
#include <fstream>
#include <regex>
#include <unistd.h>

#include "ngraph/serializer.hpp"
#include "test_util.hpp"

using namespace std;
using namespace ngraph;

namespace
{
    string golden(const string& file)
    {
        // the test binary lives in ngraph_amd/host/, the fixtures in tests/golden/serialized/
        char buf[4096];
        ssize_t n = ::readlink("/proc/self/exe", buf, sizeof buf - 1);
        string exe = n > 0 ? string(buf, static_cast<size_t>(n)) : string();
        string dir = exe.substr(0, exe.find_last_of('/'));
        return dir + "/../../tests/golden/serialized/" + file;
    }

    string slurp(const string& path)
    {
        ifstream in(path, ios::binary);
        if (!in)
            throw runtime_error("cannot open " + path);
        stringstream ss;
        ss << in.rdbuf();
        return ss.str();
    }

    // node names carry a process-wide instance number: renumber them in order of first appearance.
    // A node read from a file keeps the file's name as its friendly name (serializer.cpp:2594-2601),
    // which the writer then emits: dropped here, it is the one key a round trip adds.
    string normalize_names(const string& compact_json)
    {
        static const regex friendly_re("\"friendly_name\":\"[^\"]*\",");
        string json = regex_replace(compact_json, friendly_re, "");
        static const regex name_re("\"([A-Za-z]+)_([0-9]+)(_[0-9]+)?\"");
        map<string, string> renamed;
        string out;
        auto begin = sregex_iterator(json.begin(), json.end(), name_re);
        size_t last = 0;
        for (auto it = begin; it != sregex_iterator(); ++it)
        {
            const smatch& m = *it;
            string key = m[1].str() + "_" + m[2].str();
            if (!renamed.count(key))
                renamed[key] = m[1].str() + "#" + to_string(renamed.size());
            out += json.substr(last, static_cast<size_t>(m.position()) - last);
            out += "\"" + renamed[key] + m[3].str() + "\"";
            last = static_cast<size_t>(m.position() + m.length());
        }
        out += json.substr(last);
        return out;
    }

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
}

// ---------------------------------------------------------------------------------- reader, CPU
CPU_TEST(serializer, reads_quantized_convolution_graph)
{
    auto f = deserialize(golden("qconv_i32_output.json"));
    EXPECT_EQ(f->get_name(), string("Function_0"));
    EXPECT_EQ(f->get_parameters().size(), size_t(5));
    EXPECT_EQ(f->get_results().size(), size_t(1));
    EXPECT_EQ(count_ops_of_type<op::v0::Constant>(f), size_t(3));
    auto cv = only<op::v0::QuantizedConvolution>(f);
    EXPECT_EQ(cv->get_output_element_type(0), element::i32);
    EXPECT_EQ(cv->get_output_shape(0), (Shape{1, 1, 3, 4}));
    EXPECT_EQ(cv->get_window_movement_strides(), (Strides{1, 1}));
    EXPECT_EQ(cv->get_window_dilation_strides(), (Strides{1, 1}));
    EXPECT_EQ(cv->get_padding_below(), (CoordinateDiff{1, 1}));
    EXPECT_EQ(cv->get_padding_above(), (CoordinateDiff{1, 1}));
    EXPECT_EQ(cv->get_data_dilation_strides(), (Strides{1, 1}));
    EXPECT_TRUE(cv->get_input_axes().empty() && cv->get_filter_axes().empty() && cv->get_output_axes().empty());
    // inputs 0 / 1 are the first two parameters, in the order of the "parameters" list
    EXPECT_TRUE(cv->get_argument(0) == f->get_parameters()[0]);
    EXPECT_TRUE(cv->get_argument(1) == f->get_parameters()[1]);
    EXPECT_TRUE(cv->get_argument(2) == f->get_parameters()[2]);
    EXPECT_TRUE(is_type<op::v0::Constant>(cv->get_argument(3)));
    EXPECT_EQ(cv->get_argument(3)->get_output_element_type(0), element::u8);
    EXPECT_EQ(cv->get_argument(7)->get_output_element_type(0), element::i32);
    // names of the file survive as friendly names
    EXPECT_EQ(cv->get_friendly_name(), string("QuantizedConvolution_8"));
    EXPECT_EQ(f->get_parameters()[3]->get_friendly_name(), string("Parameter_4"));
}

CPU_TEST(serializer, reads_quantized_dot_and_quantize_graphs)
{
    auto f = deserialize(golden("qdot_u8u8.json"));
    auto qd = only<op::v0::QuantizedDot>(f);
    EXPECT_EQ(qd->get_reduction_axes_count(), size_t(1));
    EXPECT_EQ(qd->get_output_element_type(0), element::u8);
    EXPECT_EQ(qd->get_output_shape(0), (Shape{1, 3}));
    auto scale = as_type_ptr<op::v0::Constant>(qd->get_argument(2));
    EXPECT_TRUE(scale != nullptr);
    EXPECT_VEC_EQ((vector<float>{2.0f}), scale->get_vector<float>());

    auto g = deserialize(golden("quantize_dequantize.json"));
    EXPECT_EQ(g->get_results().size(), size_t(2));
    auto q = only<op::v0::Quantize>(g);
    EXPECT_TRUE(q->get_round_mode() == op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
    EXPECT_TRUE(q->get_axes().empty());
    EXPECT_EQ(q->get_output_element_type(0), element::u8);
    auto dq = only<op::v0::Dequantize>(g);
    EXPECT_EQ(dq->get_output_element_type(0), element::f32);
    EXPECT_TRUE(dq->get_argument(0) == q);
    EXPECT_EQ(g->get_output_element_type(0), element::u8);
    EXPECT_EQ(g->get_output_element_type(1), element::f32);
}

CPU_TEST(serializer, reads_legacy_layout)
{
    // no "op_version", element types as objects, opset-0 binary ops, results named directly
    auto f = deserialize(golden("legacy_scale_subgraph.json"));
    EXPECT_EQ(f->get_results().size(), size_t(1));
    EXPECT_EQ(count_ops_of_type<op::v1::Maximum>(f), size_t(1));
    EXPECT_EQ(count_ops_of_type<op::v1::Divide>(f), size_t(1));
    EXPECT_EQ(count_ops_of_type<op::v1::Add>(f), size_t(1));
    EXPECT_EQ(count_ops_of_type<op::v1::Multiply>(f), size_t(1));
    auto bc = only<op::v0::Broadcast>(f);
    EXPECT_EQ(bc->get_broadcast_shape(), (Shape{2, 3}));
    EXPECT_EQ(bc->get_broadcast_axes(), (AxisSet{0, 1}));
    EXPECT_TRUE(only<op::v1::Divide>(f)->is_pythondiv());
    // the reader put a Result on top of the named output
    EXPECT_TRUE(is_type<op::v1::Multiply>(f->get_results()[0]->get_argument(0)));
}

CPU_TEST(serializer, reads_large_constant)
{
    auto f = deserialize(golden("qconv_3x3_64ch_b128.json"));
    auto cv = only<op::v0::QuantizedConvolution>(f);
    EXPECT_EQ(cv->get_output_shape(0), (Shape{128, 64, 56, 56}));
    auto w = as_type_ptr<op::v0::Constant>(cv->get_argument(1));
    EXPECT_TRUE(w != nullptr);
    auto values = w->get_vector<int8_t>();
    EXPECT_EQ(values.size(), size_t(64 * 64 * 9));
    int lo = 0, hi = 0;
    for (int8_t v : values)
        lo = min<int>(lo, v), hi = max<int>(hi, v);
    EXPECT_EQ(lo, -127);
    EXPECT_EQ(hi, 127);
    auto s = as_type_ptr<op::v0::Constant>(cv->get_argument(2));
    EXPECT_VEC_EQ((vector<float>{0.02f}), s->get_vector<float>());
}

// ---------------------------------------------------------------------------------- writer, CPU
CPU_TEST(serializer, round_trip_is_stable)
{
    for (const char* file : {"qconv_i32_output.json", "qdot_u8u8.json", "qdot_i32_output.json", "quantize_dequantize.json", "legacy_scale_subgraph.json"})
    {
        auto f = deserialize(golden(file));
        string once = serialize(f);
        string twice = serialize(deserialize(once));
        EXPECT_EQ(normalize_names(once), normalize_names(twice));
        // pretty-printed text carries the same graph
        string pretty = serialize(f, 4);
        EXPECT_TRUE(pretty.find('\n') != string::npos);
        EXPECT_EQ(normalize_names(serialize(deserialize(pretty))), normalize_names(once));
    }
    // for a file in the current layout the text itself comes back (same keys, same order, same values)
    string text = slurp(golden("qdot_u8u8.json"));
    EXPECT_EQ(normalize_names(serialize(deserialize(text))), normalize_names(text));
}

CPU_TEST(serializer, writes_every_op_of_the_path)
{
    // one graph through every op the writer knows, built with the C++ API, read back and compared
    auto X = make_shared<op::v0::Parameter>(element::f32, Shape{2, 4, 6, 6});
    auto scale = op::v0::Constant::create(element::f32, Shape{4}, {0.5f, 0.25f, 1.0f, 2.0f});
    auto zp = op::v0::Constant::create(element::u8, Shape{4}, {1, 2, 3, 4});
    auto q = make_shared<op::v0::Quantize>(X, scale, zp, element::u8, AxisSet{1}, op::v0::Quantize::RoundMode::ROUND_NEAREST_UPWARD);
    auto mp = make_shared<op::v0::MaxPool>(q, Shape{2, 2}, Strides{2, 2}, Shape{0, 0}, Shape{0, 0});
    auto ap = make_shared<op::v0::AvgPool>(q, Shape{2, 2}, Strides{2, 2}, Shape{0, 0}, Shape{0, 0}, true);
    auto cat = make_shared<op::v0::Concat>(OutputVector{mp, ap}, 1);
    auto dq_scale = op::v0::Constant::create(element::f32, Shape{}, {0.125f});
    auto dq_zp = op::v0::Constant::create(element::u8, Shape{}, {0});
    auto dq = make_shared<op::v0::Dequantize>(cat, dq_scale, dq_zp, element::f32, AxisSet{});
    auto rs = make_shared<op::v0::Reshape>(dq, AxisVector{0, 2, 3, 1}, Shape{18, 8});
    auto relu = make_shared<op::v0::Relu>(rs);
    auto ab = make_shared<op::v0::Abs>(relu);
    auto sm = make_shared<op::v0::Softmax>(ab, AxisSet{1});
    auto ln = make_shared<op::v0::LayerNorm>(sm, false, 1, 1e-5);
    auto ge = make_shared<op::v0::Gelu>(ln);
    auto er = make_shared<op::v0::Erf>(ge);
    auto c3 = op::v0::Constant::create(element::f32, Shape{}, {3.0f});
    auto bc = make_shared<op::v0::Broadcast>(c3, Shape{18, 8}, AxisSet{0, 1});
    auto add = make_shared<op::v1::Add>(er, bc);
    auto sub = make_shared<op::v1::Subtract>(add, bc);
    auto mul = make_shared<op::v1::Multiply>(sub, bc);
    auto div = make_shared<op::v1::Divide>(mul, bc, false);
    auto mx = make_shared<op::v1::Maximum>(div, bc);
    auto mn = make_shared<op::v1::Minimum>(mx, bc);
    auto cvt = make_shared<op::v0::Convert>(mn, element::i32);
    auto f = make_shared<Function>(OutputVector{cvt}, ParameterVector{X}, "every_op");

    string text = serialize(f);
    auto g = deserialize(text);
    EXPECT_EQ(g->get_name(), string("every_op"));
    auto fo = f->get_ordered_ops(), go = g->get_ordered_ops();
    EXPECT_EQ(fo.size(), go.size());
    for (size_t i = 0; i < min(fo.size(), go.size()); ++i)
    {
        EXPECT_TRUE(fo[i]->get_type_info() == go[i]->get_type_info());
        EXPECT_EQ(fo[i]->get_output_size(), go[i]->get_output_size());
        EXPECT_EQ(fo[i]->get_output_shape(0), go[i]->get_output_shape(0));
        EXPECT_EQ(fo[i]->get_output_element_type(0), go[i]->get_output_element_type(0));
        EXPECT_EQ(go[i]->get_friendly_name(), fo[i]->get_name());
    }
    auto q2 = only<op::v0::Quantize>(g);
    EXPECT_TRUE(q2->get_round_mode() == op::v0::Quantize::RoundMode::ROUND_NEAREST_UPWARD);
    EXPECT_EQ(q2->get_axes(), (AxisSet{1}));
    EXPECT_VEC_EQ((vector<float>{0.5f, 0.25f, 1.0f, 2.0f}), as_type_ptr<op::v0::Constant>(q2->get_argument(1))->get_vector<float>());
    EXPECT_VEC_EQ((vector<uint8_t>{1, 2, 3, 4}), as_type_ptr<op::v0::Constant>(q2->get_argument(2))->get_vector<uint8_t>());
    EXPECT_TRUE(only<op::v0::AvgPool>(g)->get_include_padding_in_avg_computation());
    EXPECT_EQ(only<op::v0::Reshape>(g)->get_input_order(), (AxisVector{0, 2, 3, 1}));
    EXPECT_FALSE(only<op::v1::Divide>(g)->is_pythondiv());
    EXPECT_FALSE(only<op::v0::LayerNorm>(g)->get_use_affine());
    EXPECT_EQ(only<op::v0::Softmax>(g)->get_axes(), (AxisSet{1}));
    EXPECT_EQ(only<op::v0::Concat>(g)->get_concatenation_axis(), int64_t(1));
    EXPECT_EQ(normalize_names(serialize(g)), normalize_names(text));
    // the opset-1 binary ops take nGraph's attribute-visitor spelling
    EXPECT_TRUE(text.find("\"attribute_visitor\":true") != string::npos);
    EXPECT_TRUE(text.find("\"m_pythondiv\":false") != string::npos);
}

CPU_TEST(serializer, constant_literals)
{
    // reals are written with max_digits10 digits and read back bit for bit; NAN / INFINITY spellings;
    // a tensor of one repeated value is written as a single literal (serializer.cpp:2852-2869)
    vector<float> vals = {0.1f, -3.4028235e38f, 1.17549435e-38f, 1e-45f, 16777217.0f, -0.0f};
    auto c = op::v0::Constant::create(element::f32, Shape{6}, vals);
    auto inf = make_shared<op::v0::Constant>(element::f32, Shape{3}, vector<float>{INFINITY, -INFINITY, NAN});
    auto same = op::v0::Constant::create(element::i8, Shape{2, 3}, {-7});
    auto big = op::v0::Constant::create(element::i32, Shape{2}, {2147483647, -2147483647 - 1});
    auto f = make_shared<Function>(OutputVector{c, inf, same, big}, ParameterVector{});
    string text = serialize(f);
    EXPECT_TRUE(text.find("\"value\":[\"-7\"]") != string::npos);
    EXPECT_TRUE(text.find("\"INFINITY\",\"-INFINITY\",\"NAN\"") != string::npos);
    EXPECT_TRUE(text.find("\"0.100000001\"") != string::npos);
    auto g = deserialize(text);
    vector<shared_ptr<op::v0::Constant>> cs;
    for (const auto& r : g->get_results())
        cs.push_back(as_type_ptr<op::v0::Constant>(r->get_argument(0)));
    auto back = cs[0]->get_vector<float>();
    EXPECT_EQ(memcmp(back.data(), vals.data(), vals.size() * sizeof(float)), 0);
    auto inf_back = cs[1]->get_vector<float>();
    EXPECT_TRUE(isinf(inf_back[0]) && inf_back[0] > 0 && isinf(inf_back[1]) && inf_back[1] < 0 && isnan(inf_back[2]));
    EXPECT_VEC_EQ((vector<int8_t>{-7, -7, -7, -7, -7, -7}), cs[2]->get_vector<int8_t>());
    EXPECT_VEC_EQ((vector<int32_t>{2147483647, -2147483647 - 1}), cs[3]->get_vector<int32_t>());
}

// ---------------------------------------------------------------------------------- errors, CPU
CPU_TEST(serializer, error_messages)
{
    // an op outside the path stops the reader with nGraph's message (serializer.cpp:2616-2630, 2577-2581)
    string sigmoid = R"([{"name":"F","ops":[{"element_type":"float","inputs":[],"name":"Parameter_0","op":"Parameter","outputs":["Parameter_0_0"],"shape":[3,4]},
        {"inputs":["Parameter_0"],"name":"Negative_3","op":"Negative","outputs":["Negative_3_0"]}],"parameters":["Parameter_0"],"result":["Negative_3"]}])";
    string msg = what_of([&] { deserialize(sigmoid); });
    EXPECT_TRUE(msg.find("Error parsing json at node 'Negative_3'") == 0);
    EXPECT_TRUE(msg.find("unsupported op Negative:0") != string::npos);
    // the fused quantized ops have no JSON form in nGraph either
    string fused = R"([{"name":"F","ops":[{"name":"QuantizedConvolutionBias_1","op":"QuantizedConvolutionBias","op_version":0,"inputs":[]}],"parameters":[],"result":[]}])";
    EXPECT_TRUE(what_of([&] { deserialize(fused); }).find("unsupported op QuantizedConvolutionBias:0") != string::npos);
    // references to nodes that were never defined, missing attributes, wrong literal counts
    string dangling = R"([{"name":"F","ops":[{"name":"Relu_1","op":"Relu","op_version":0,"inputs":["Parameter_9"]}],"parameters":[],"result":["Relu_1"]}])";
    EXPECT_TRUE(what_of([&] { deserialize(dangling); }).find("Error parsing json at node 'Relu_1'") == 0);
    string no_axes = R"([{"name":"F","ops":[{"element_type":"float","name":"P","op":"Parameter","shape":[2]},{"element_type":"float","name":"S","op":"Constant","shape":[],"value":["1"]},
        {"element_type":"int8_t","name":"Z","op":"Constant","shape":[],"value":["0"]},{"name":"Q","op":"Quantize","inputs":["P","S","Z"],"type":"int8_t","round_mode":4}],"parameters":["P"],"result":["Q"]}])";
    EXPECT_TRUE(what_of([&] { deserialize(no_axes); }).find("key 'axes' not found") != string::npos);
    string bad_count = R"([{"name":"F","ops":[{"element_type":"float","name":"C","op":"Constant","shape":[3],"value":["1","2"]}],"parameters":[],"result":["C"]}])";
    EXPECT_TRUE(what_of([&] { deserialize(bad_count); }).find("expected number of literals") != string::npos);
    string bad_literal = R"([{"name":"F","ops":[{"element_type":"int8_t","name":"C","op":"Constant","shape":[1],"value":["12x"]}],"parameters":[],"result":["C"]}])";
    EXPECT_TRUE(what_of([&] { deserialize(bad_literal); }).find("Could not parse literal '12x'") != string::npos);
    // Results on some outputs only (serializer.cpp:838-842)
    string mixed = R"([{"name":"F","ops":[{"element_type":"float","name":"P","op":"Parameter","shape":[2]},{"name":"R","op":"Result","inputs":["P"]},{"name":"A","op":"Abs","inputs":["P"]}],
        "parameters":["P"],"result":["R","A"]}])";
    EXPECT_TRUE(what_of([&] { deserialize(mixed); }).find("Some op::v0::Results appear to be missing") != string::npos);
    // dynamic shapes are outside this backend
    string dyn = R"([{"name":"F","ops":[{"element_type":"float","name":"P","op":"Parameter","shape":[2,null]}],"parameters":["P"],"result":["P"]}])";
    EXPECT_TRUE(what_of([&] { deserialize(dyn); }).find("dynamic dimensions") != string::npos);
    // cpio containers are told apart from json and refused
    EXPECT_TRUE(what_of([&] { deserialize(string("\x71\xC7 rest")); }).find("cpio") != string::npos);
    EXPECT_TRUE(what_of([&] { deserialize(string("070707000000")); }).find("cpio") != string::npos);
}

CPU_TEST(serializer, json_text)
{
    // malformed text: position in the message, no crash
    for (const char* bad : {"", "[", "[{]", "[{\"name\":}]", "[{\"a\":1,}]", "[1 2]", "[\"abc]", "[\"\\q\"]", "[\"\\u12\"]", "[\"\\ud800\"]", "[01]", "[1.]", "[1e]", "[-]", "[tru]",
                            "[{\"a\":1}] x", "{\"a\":\"\x01\"}"})
    {
        string msg = what_of([&] { deserialize(string(bad)); });
        EXPECT_TRUE(msg.find("json parse error at line") == 0);
    }
    // nesting beyond the parser's limit is an error, not a stack overflow
    EXPECT_TRUE(what_of([&] { deserialize(string(100000, '[')); }).find("nesting deeper") != string::npos);
    // escapes, unicode and whitespace in a well-formed file; unknown keys are ignored; numbers as reals
    string ok = "\t[ {\r\n \"name\" : \"f\\u00e9\\n\\\"\\\\\\/\\ud83d\\ude00\", \"extra\" : {\"x\":[1,2.5e0,-3E+2,null,true]},\n"
                " \"ops\":[{\"element_type\":\"float\",\"name\":\"P\",\"friendly_name\":\"in\\tput\",\"op\":\"Parameter\",\"shape\":[2.0,3]}],"
                " \"parameters\":[\"P\"], \"result\":[\"P\"] } ]  ";
    auto f = deserialize(ok);
    EXPECT_EQ(f->get_name(), string("f\xC3\xA9\n\"\\/\xF0\x9F\x98\x80"));
    EXPECT_EQ(f->get_parameters()[0]->get_output_shape(0), (Shape{2, 3}));
    EXPECT_EQ(f->get_parameters()[0]->get_friendly_name(), string("in\tput"));
    // and the writer escapes what it must
    string text = serialize(f);
    EXPECT_TRUE(text.find("in\\tput") != string::npos);
    EXPECT_EQ(deserialize(text)->get_name(), f->get_name());
    // the last function of a file is the one returned (serializer.cpp:518-521)
    string two = R"([{"name":"first","ops":[{"element_type":"float","name":"P","op":"Parameter","shape":[1]}],"parameters":["P"],"result":["P"]},
                     {"name":"second","ops":[{"element_type":"float","name":"P","op":"Parameter","shape":[2]}],"parameters":["P"],"result":["P"]}])";
    EXPECT_EQ(deserialize(two)->get_name(), string("second"));
    // streams and file names
    stringstream ss(two);
    EXPECT_EQ(deserialize(ss)->get_name(), string("second"));
    string path = "/tmp/hipq_serializer_test_" + to_string(::getpid()) + ".json";
    serialize(path, f, 2);
    EXPECT_EQ(deserialize(path)->get_name(), f->get_name());
    ::unlink(path.c_str());
}

// ---------------------------------------------------------------------------------- loaded graphs on the device
GPU_TEST(serializer, quantized_conv_int32_output_from_json)
{
    auto f = deserialize(golden("qconv_i32_output.json"));
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor(element::u8, Shape{1, 1, 3, 4});
    copy_data(a, vector<uint8_t>{1, 2, 3, 4, 5, 6, 7, 0, 1, 2, 3, 4});
    auto b = backend->create_tensor(element::u8, Shape{1, 1, 3, 3});
    copy_data(b, vector<uint8_t>{1, 2, 3, 4, 5, 0, 0, 1, 2});
    vector<shared_ptr<runtime::Tensor>> inputs{a, b};
    for (int i = 0; i < 3; ++i)
    {
        auto t = backend->create_tensor(element::f32, Shape{});
        copy_data(t, vector<float>{1.0f});
        inputs.push_back(t);
    }
    auto result = backend->create_tensor(element::i32, Shape{1, 1, 3, 4});
    auto handle = backend->compile(f);
    handle->call_with_validate({result}, inputs);
    EXPECT_VEC_EQ((vector<int32_t>{22, 34, 30, 32, 38, 72, 90, 43, 33, 52, 43, 39}), read_vector<int32_t>(result));
    // and after a trip through this library's writer
    auto g = deserialize(serialize(f, 2));
    auto result2 = backend->create_tensor(element::i32, Shape{1, 1, 3, 4});
    backend->compile(g)->call_with_validate({result2}, inputs);
    EXPECT_VEC_EQ(read_vector<int32_t>(result), read_vector<int32_t>(result2));
}

GPU_TEST(serializer, quantized_dot_from_json)
{
    auto backend = runtime::Backend::create("HIP");
    {
        auto f = deserialize(golden("qdot_u8u8.json"));
        auto a = backend->create_tensor(element::u8, Shape{1, 2});
        copy_data(a, vector<uint8_t>{2, 3});
        auto b = backend->create_tensor(element::u8, Shape{2, 3});
        copy_data(b, vector<uint8_t>{0, 2, 4, 1, 3, 5});
        auto result = backend->create_tensor(element::u8, Shape{1, 3});
        backend->compile(f)->call_with_validate({result}, {a, b});
        EXPECT_VEC_EQ((vector<uint8_t>{3, 13, 23}), read_vector<uint8_t>(result));
    }
    {
        auto f = deserialize(golden("qdot_i32_output.json"));
        auto a = backend->create_tensor(element::u8, Shape{1, 2});
        copy_data(a, vector<uint8_t>{2, 3});
        auto b = backend->create_tensor(element::i8, Shape{2, 3});
        copy_data(b, vector<int8_t>{0, 1, 2, 3, 4, 5});
        auto result = backend->create_tensor(element::i32, Shape{1, 3});
        backend->compile(f)->call_with_validate({result}, {a, b});
        EXPECT_VEC_EQ((vector<int32_t>{9, 14, 19}), read_vector<int32_t>(result));
    }
}

GPU_TEST(serializer, quantize_dequantize_from_json)
{
    auto f = deserialize(golden("quantize_dequantize.json"));
    auto backend = runtime::Backend::create("HIP");
    auto x = backend->create_tensor(element::f32, Shape{4, 3});
    copy_data(x, vector<float>{0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11});
    auto q = backend->create_tensor(element::u8, Shape{4, 3});
    auto dq = backend->create_tensor(element::f32, Shape{4, 3});
    backend->compile(f)->call_with_validate({q, dq}, {x});
    EXPECT_VEC_EQ((vector<uint8_t>{1, 1, 2, 3, 3, 3, 4, 5, 5, 5, 6, 7}), read_vector<uint8_t>(q));
    EXPECT_VEC_EQ((vector<float>{0, 0, 2, 4, 4, 4, 6, 8, 8, 8, 10, 12}), read_vector<float>(dq));
}

GPU_TEST(serializer, legacy_float_glue_from_json)
{
    auto f = deserialize(golden("legacy_scale_subgraph.json"));
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor(element::f32, Shape{2, 3});
    copy_data(a, vector<float>{-1, 2, -3, 4, -5, 6});
    auto b = backend->create_tensor(element::f32, Shape{2, 3});
    copy_data(b, vector<float>{0.5f, 0.5f, 8, 1, 1, 1});
    auto r = backend->create_tensor(element::f32, Shape{2, 3});
    backend->compile(f)->call_with_validate({r}, {a, b});
    // (max(|a|, b) / 2 + a) * b, every step exact in binary32
    EXPECT_VEC_EQ((vector<float>{-0.25f, 1.5f, 8.0f, 6.0f, -2.5f, 9.0f}), read_vector<float>(r));
}

// the headline layer loaded from JSON gives the bytes of the same graph built through the C++ API
GPU_TEST(serializer, headline_layer_from_json_matches_api_built_graph)
{
    auto f = deserialize(golden("qconv_3x3_64ch_b128.json"));
    auto cv = only<op::v0::QuantizedConvolution>(f);
    auto w = as_type_ptr<op::v0::Constant>(cv->get_argument(1));
    const size_t batch = 4; // same graph at a batch a host comparison finishes quickly
    auto X = make_shared<op::v0::Parameter>(element::u8, Shape{batch, 64, 56, 56});
    auto W = make_shared<op::v0::Constant>(element::i8, Shape{64, 64, 3, 3}, w->get_data_ptr());
    auto c = [](const element::Type& t, double v) { return op::v0::Constant::create(t, Shape{}, {v}); };
    auto api = make_shared<op::v0::QuantizedConvolution>(X, W, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{1, 1}, CoordinateDiff{1, 1}, Strides{1, 1},
                                                         c(element::f32, 0.02f), c(element::u8, 0), c(element::f32, 0.005f), c(element::i8, 0),
                                                         c(element::f32, 0.1f), c(element::i8, 0), element::i8);
    auto f_api = make_shared<Function>(OutputVector{api}, ParameterVector{X});
    // the JSON graph re-batched through its own text: only the Parameter's and nothing else changes
    string text = serialize(f);
    size_t at = text.find("[128,64,56,56]");
    EXPECT_TRUE(at != string::npos);
    text.replace(at, strlen("[128,64,56,56]"), "[4,64,56,56]");
    auto f_json = deserialize(text);

    auto backend = runtime::Backend::create("HIP");
    vector<uint8_t> data(batch * 64 * 56 * 56);
    uint32_t state = 12345;
    for (auto& v : data)
    {
        state = state * 1664525u + 1013904223u;
        v = static_cast<uint8_t>(state >> 24);
    }
    auto x = backend->create_tensor(element::u8, Shape{batch, 64, 56, 56});
    copy_data(x, data);
    auto y_json = backend->create_tensor(element::i8, Shape{batch, 64, 56, 56});
    auto y_api = backend->create_tensor(element::i8, Shape{batch, 64, 56, 56});
    backend->compile(f_json)->call_with_validate({y_json}, {x});
    backend->compile(f_api)->call_with_validate({y_api}, {x});
    auto got = read_vector<int8_t>(y_json), expect = read_vector<int8_t>(y_api);
    EXPECT_TRUE(got == expect);
    size_t nonzero = 0;
    for (int8_t v : got)
        nonzero += v != 0;
    EXPECT_TRUE(nonzero > got.size() / 2);
}
