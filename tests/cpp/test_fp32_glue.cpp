// Softmax / Erf / Gelu / LayerNorm / BatchMatMul / BatchMatMulTranspose through backend "HIP", with
// the values of the reference's test/backend/softmax.in.cpp:66-221, erf.in.cpp:47-66,
// gelu.in.cpp:49-108, layer_norm.in.cpp:48-91 and batch_mat_mul.in.cpp:51-102; type propagation
// after src/ngraph/op/{softmax,gelu,layer_norm}.cpp and op/experimental/batch_mat_mul.cpp.
#include <cmath>
#include <cstdlib>
#include <set>

#include "test_util.hpp"

using namespace std;
using namespace ngraph;

namespace
{
    bool close(const vector<float>& a, const vector<float>& b, float rtol = 1e-5f, float atol = 1e-7f)
    {
        if (a.size() != b.size())
            return false;
        for (size_t i = 0; i < a.size(); ++i)
            if (!(fabs(a[i] - b[i]) <= atol + rtol * fabs(b[i])))
                return false;
        return true;
    }

    vector<float> run(const shared_ptr<Function>& f, const vector<pair<Shape, vector<float>>>& args, const Shape& out_shape)
    {
        auto backend = runtime::Backend::create("HIP");
        vector<shared_ptr<runtime::Tensor>> in;
        for (const auto& a : args)
        {
            in.push_back(backend->create_tensor(element::f32, a.first));
            copy_data(in.back(), a.second);
        }
        auto result = backend->create_tensor(element::f32, out_shape);
        auto handle = backend->compile(f);
        handle->call_with_validate({result}, in);
        return read_vector<float>(result);
    }
}

GPU_TEST(HIP, softmax_all_and_empty_axis_set)
{
    Shape shape{2, 3};
    const vector<float> x{-3, -2, -1, 0, 1, 2};
    const float d = expf(-3) + expf(-2) + expf(-1) + expf(0) + expf(1) + expf(2);
    const vector<float> expected{expf(-3) / d, expf(-2) / d, expf(-1) / d, expf(0) / d, expf(1) / d, expf(2) / d};
    for (const AxisSet& axes : {AxisSet{0, 1}, AxisSet{}})
    {
        auto A = make_shared<op::v0::Parameter>(element::f32, shape);
        auto f = make_shared<Function>(OutputVector{make_shared<op::v0::Softmax>(A, axes)}, ParameterVector{A});
        EXPECT_TRUE(close(run(f, {{shape, x}}, shape), expected));
    }
}

GPU_TEST(HIP, softmax_axis_3d)
{
    Shape shape{2, 2, 3};
    const vector<float> x{-10, -20, -30, -40, -50, -60, -1, -2, -3, -4, -5, -6};
    auto A = make_shared<op::v0::Parameter>(element::f32, shape);
    auto f = make_shared<Function>(OutputVector{make_shared<op::v0::Softmax>(A, AxisSet{0})}, ParameterVector{A});
    vector<float> expected(12);
    for (int i = 0; i < 6; ++i)
    {
        const float d = expf(x[i]) + expf(x[i + 6]);
        expected[i] = expf(x[i]) / d;
        expected[i + 6] = expf(x[i + 6]) / d;
    }
    EXPECT_TRUE(close(run(f, {{shape, x}}, shape), expected, 1e-5f, 1e-8f));
}

GPU_TEST(HIP, softmax_axis_rows_and_columns)
{
    Shape shape{2, 3};
    const vector<float> x{-10, -20, -30, -40, -50, -60};
    {
        auto A = make_shared<op::v0::Parameter>(element::f32, shape);
        auto f = make_shared<Function>(OutputVector{make_shared<op::v0::Softmax>(A, AxisSet{1})}, ParameterVector{A});
        const float d0 = expf(-10) + expf(-20) + expf(-30), d1 = expf(-40) + expf(-50) + expf(-60);
        EXPECT_TRUE(close(run(f, {{shape, x}}, shape), {expf(-10) / d0, expf(-20) / d0, expf(-30) / d0, expf(-40) / d1, expf(-50) / d1, expf(-60) / d1}));
    }
    {
        auto A = make_shared<op::v0::Parameter>(element::f32, shape);
        auto f = make_shared<Function>(OutputVector{make_shared<op::v0::Softmax>(A, AxisSet{0})}, ParameterVector{A});
        const float d0 = expf(-10) + expf(-40), d1 = expf(-20) + expf(-50), d2 = expf(-30) + expf(-60);
        EXPECT_TRUE(close(run(f, {{shape, x}}, shape), {expf(-10) / d0, expf(-20) / d1, expf(-30) / d2, expf(-40) / d0, expf(-50) / d1, expf(-60) / d2}));
    }
}

GPU_TEST(HIP, erf_and_gelu)
{
    Shape shape{4096};
    vector<float> x(4096), e(4096), g(4096);
    for (size_t i = 0; i < x.size(); ++i)
    {
        x[i] = -100.0f + 200.0f * static_cast<float>((i * 2654435761u) % 100003) / 100003.0f;
        if (i % 2)
            x[i] *= 0.03f; // half of the points where erf is not saturated
        e[i] = erff(x[i]);
        g[i] = 0.5f * x[i] * (1.0f + erff(x[i] / sqrtf(2.0f)));
    }
    auto A = make_shared<op::v0::Parameter>(element::f32, shape);
    auto fe = make_shared<Function>(OutputVector{make_shared<op::v0::Erf>(A)}, ParameterVector{A});
    EXPECT_TRUE(close(run(fe, {{shape, x}}, shape), e, 1e-6f, 3e-7f));
    auto B = make_shared<op::v0::Parameter>(element::f32, shape);
    auto fg = make_shared<Function>(OutputVector{make_shared<op::v0::Gelu>(B)}, ParameterVector{B});
    // the reference's own tolerance for this op (test/backend/gelu.in.cpp:78) and a tighter one
    auto got = run(fg, {{shape, x}}, shape);
    EXPECT_TRUE(close(got, g, .007f, .007f));
    EXPECT_TRUE(close(got, g, 1e-5f, 3e-5f));
}

GPU_TEST(HIP, layer_norm_affine)
{
    // layer_norm_affine_stats of the reference without the statistics outputs
    auto data = make_shared<op::v0::Parameter>(element::f32, Shape{2, 4});
    auto scale = make_shared<op::v0::Parameter>(element::f32, Shape{4});
    auto bias = make_shared<op::v0::Parameter>(element::f32, Shape{4});
    auto ln = make_shared<op::v0::LayerNorm>(data, scale, bias, false);
    auto f = make_shared<Function>(OutputVector{ln}, ParameterVector{data, scale, bias});
    auto got = run(f, {{Shape{2, 4}, {-4, -3, -2, -1, 0, 1, 2, 3}}, {Shape{4}, {-1, 1, 2, 3}}, {Shape{4}, {-4, -3, -2, -1}}}, Shape{2, 4});
    const vector<float> expected{-2.658364534378051758f, -3.447211742401123047f, -1.105576276779174805f, 3.024906158447265625f,
                                 -2.658364534378051758f, -3.447211742401123047f, -1.105576276779174805f, 3.024906158447265625f};
    EXPECT_TRUE(close(got, expected, 1e-5f, 1e-6f));
    // without affine, normalising the last axis of a 3-D tensor
    auto d3 = make_shared<op::v0::Parameter>(element::f32, Shape{1, 2, 4});
    auto f3 = make_shared<Function>(OutputVector{make_shared<op::v0::LayerNorm>(d3, false, -1)}, ParameterVector{d3});
    auto n3 = run(f3, {{Shape{1, 2, 4}, {-4, -3, -2, -1, 0, 1, 2, 3}}}, Shape{1, 2, 4});
    const float sd = sqrtf(1.25f + 1e-5f);
    EXPECT_TRUE(close(n3, {-1.5f / sd, -0.5f / sd, 0.5f / sd, 1.5f / sd, -1.5f / sd, -0.5f / sd, 0.5f / sd, 1.5f / sd}, 1e-5f, 1e-6f));
}

GPU_TEST(HIP, layer_norm_affine_stats)
{
    // test/backend/layer_norm.in.cpp:48-91: three outputs
    auto p_data = make_shared<op::v0::Parameter>(element::f32, Shape{2, 4});
    auto p_scale = make_shared<op::v0::Parameter>(element::f32, Shape{4});
    auto p_bias = make_shared<op::v0::Parameter>(element::f32, Shape{4});
    auto ln = make_shared<op::v0::LayerNorm>(p_data, p_scale, p_bias);
    EXPECT_EQ(ln->get_output_size(), size_t(3));
    auto f = make_shared<Function>(OutputVector{ln->output(0), ln->output(1), ln->output(2)}, ParameterVector{p_data, p_scale, p_bias});
    auto backend = runtime::Backend::create("HIP");
    auto data = backend->create_tensor(element::f32, Shape{2, 4});
    auto scale = backend->create_tensor(element::f32, Shape{4});
    auto bias = backend->create_tensor(element::f32, Shape{4});
    copy_data(data, vector<float>{-4, -3, -2, -1, 0, 1, 2, 3});
    copy_data(scale, vector<float>{-1, 1, 2, 3});
    copy_data(bias, vector<float>{-4, -3, -2, -1});
    auto norm = backend->create_tensor(element::f32, Shape{2, 4});
    auto mean = backend->create_tensor(element::f32, Shape{2});
    auto var = backend->create_tensor(element::f32, Shape{2});
    auto handle = backend->compile(f);
    const vector<float> exp_norm{-2.658364534378051758f, -3.447211742401123047f, -1.105576276779174805f, 3.024906158447265625f,
                                 -2.658364534378051758f, -3.447211742401123047f, -1.105576276779174805f, 3.024906158447265625f};
    for (int rep = 0; rep < 3; ++rep) // eager, captured, replayed
    {
        handle->call_with_validate({norm, mean, var}, {data, scale, bias});
        EXPECT_TRUE(close(read_vector<float>(norm), exp_norm, 1e-5f, 1e-6f));
        EXPECT_VEC_EQ((vector<float>{-2.5f, 1.5f}), read_vector<float>(mean));
        EXPECT_VEC_EQ((vector<float>{1.25f, 1.25f}), read_vector<float>(var));
    }
    // a statistic consumed inside the graph: variance + mean
    auto d2 = make_shared<op::v0::Parameter>(element::f32, Shape{2, 4});
    auto ln2 = make_shared<op::v0::LayerNorm>(d2, true, 1);
    auto sum = make_shared<op::v1::Add>(ln2->output(1), ln2->output(2));
    auto f2 = make_shared<Function>(OutputVector{sum}, ParameterVector{d2});
    EXPECT_VEC_EQ((vector<float>{-1.25f, 2.75f}), run(f2, {{Shape{2, 4}, {-4, -3, -2, -1, 0, 1, 2, 3}}}, Shape{2}));
}

GPU_TEST(HIP, batch_mat_mul_and_transpose)
{
    const vector<float> a{1, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4, 4};
    const vector<float> b{1, 1, 1, 1, 2, 2, 2, 2, 3, 3, 3, 3, 1, 1, 1, 1, 2, 2, 2, 2, 3, 3, 3, 3};
    {
        auto A = make_shared<op::v0::Parameter>(element::f32, Shape{2, 2, 3});
        auto B = make_shared<op::v0::Parameter>(element::f32, Shape{2, 3, 4});
        auto f = make_shared<Function>(OutputVector{make_shared<op::v0::BatchMatMulTranspose>(A, B, false, false)}, ParameterVector{A, B});
        EXPECT_VEC_EQ((vector<float>{6, 6, 6, 6, 12, 12, 12, 12, 18, 18, 18, 18, 24, 24, 24, 24}), run(f, {{Shape{2, 2, 3}, a}, {Shape{2, 3, 4}, b}}, Shape{2, 2, 4}));
        auto A2 = make_shared<op::v0::Parameter>(element::f32, Shape{2, 2, 3});
        auto B2 = make_shared<op::v0::Parameter>(element::f32, Shape{2, 3, 4});
        auto f2 = make_shared<Function>(OutputVector{make_shared<op::v0::BatchMatMul>(A2, B2)}, ParameterVector{A2, B2});
        EXPECT_VEC_EQ((vector<float>{6, 6, 6, 6, 12, 12, 12, 12, 18, 18, 18, 18, 24, 24, 24, 24}), run(f2, {{Shape{2, 2, 3}, a}, {Shape{2, 3, 4}, b}}, Shape{2, 2, 4}));
    }
    {
        auto A = make_shared<op::v0::Parameter>(element::f32, Shape{2, 3, 2});
        auto B = make_shared<op::v0::Parameter>(element::f32, Shape{2, 3, 4});
        auto f = make_shared<Function>(OutputVector{make_shared<op::v0::BatchMatMulTranspose>(A, B, true, false)}, ParameterVector{A, B});
        EXPECT_VEC_EQ((vector<float>{9, 9, 9, 9, 11, 11, 11, 11, 21, 21, 21, 21, 23, 23, 23, 23}), run(f, {{Shape{2, 3, 2}, a}, {Shape{2, 3, 4}, b}}, Shape{2, 2, 4}));
    }
}

CPU_TEST(type_prop, fp32_glue_shapes_and_failures)
{
    auto x = make_shared<op::v0::Parameter>(element::f32, Shape{2, 3, 4});
    EXPECT_EQ(make_shared<op::v0::Softmax>(x, AxisSet{2})->get_output_shape(0), (Shape{2, 3, 4}));
    EXPECT_EQ(make_shared<op::v0::Softmax>(x, AxisSet{})->get_axes().size(), size_t(3));
    EXPECT_THROW(make_shared<op::v0::Softmax>(x, AxisSet{3}), NodeValidationFailure);
    auto q = make_shared<op::v0::Parameter>(element::i8, Shape{4});
    EXPECT_THROW(make_shared<op::v0::Gelu>(q), NodeValidationFailure);
    EXPECT_THROW(make_shared<op::v0::LayerNorm>(q, false), NodeValidationFailure);
    auto ln = make_shared<op::v0::LayerNorm>(x, true, 1);
    EXPECT_EQ(ln->get_output_size(), size_t(3));
    EXPECT_EQ(ln->get_output_shape(1), (Shape{2}));
    EXPECT_EQ(make_shared<op::v0::LayerNorm>(x, true, -1)->get_output_shape(2), (Shape{2, 3}));
    EXPECT_THROW(make_shared<op::v0::LayerNorm>(x, true, 3), NodeValidationFailure);
    auto s2 = make_shared<op::v0::Parameter>(element::f32, Shape{3, 4});
    auto s1 = make_shared<op::v0::Parameter>(element::f32, Shape{4});
    EXPECT_NO_THROW(make_shared<op::v0::LayerNorm>(x, s2, s2, false, 1));
    EXPECT_NO_THROW(make_shared<op::v0::LayerNorm>(x, s1, s1, false, 2));
    auto s3 = make_shared<op::v0::Parameter>(element::f32, Shape{2, 3, 4});
    EXPECT_THROW(make_shared<op::v0::LayerNorm>(x, s3, s3, false, 1), NodeValidationFailure);
    auto a = make_shared<op::v0::Parameter>(element::f32, Shape{5, 2, 3});
    auto b = make_shared<op::v0::Parameter>(element::f32, Shape{5, 3, 7});
    EXPECT_EQ(make_shared<op::v0::BatchMatMul>(a, b)->get_output_shape(0), (Shape{5, 2, 7}));
    EXPECT_EQ(make_shared<op::v0::BatchMatMulTranspose>(b, b, true, false)->get_output_shape(0), (Shape{5, 7, 7}));
    EXPECT_THROW(make_shared<op::v0::BatchMatMul>(a, a), NodeValidationFailure);
    auto c = make_shared<op::v0::Parameter>(element::f32, Shape{4, 3, 7});
    EXPECT_THROW(make_shared<op::v0::BatchMatMul>(a, c), NodeValidationFailure);
    auto m = make_shared<op::v0::Parameter>(element::f32, Shape{3, 7});
    EXPECT_THROW(make_shared<op::v0::BatchMatMul>(a, m), NodeValidationFailure);
}

// ---- glue fusion of the backend: Multiply into Softmax, Add into LayerNorm, Quantize into the
// LayerNorm / Gelu that feeds it.  Every fused launch equals the op sequence bit for bit, so the
// results with NGRAPH_PASS_ENABLES "HIPGlueFusion:0" and with the default must be identical, and the
// fused executable runs fewer launches (one performance counter a launch).
namespace
{
    struct GlueRun
    {
        vector<vector<uint8_t>> bytes; // every result, raw
        size_t launches;
    };

    GlueRun run_glue(const shared_ptr<Function>& f, const vector<vector<float>>& args, bool fuse)
    {
        setenv("NGRAPH_PASS_ENABLES", fuse ? "HIPGlueFusion:1" : "HIPGlueFusion:0", 1);
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
        auto exec = backend->compile(f, true);
        exec->call_with_validate(out, in);
        unsetenv("NGRAPH_PASS_ENABLES");
        GlueRun r;
        r.launches = exec->get_performance_data().size();
        for (auto& t : out)
        {
            vector<uint8_t> b(shape_size(t->get_shape()) * t->get_element_type().size());
            t->read(b.data(), b.size());
            r.bytes.push_back(b);
        }
        return r;
    }

    vector<float> wave(size_t n, float amplitude, float step)
    {
        vector<float> v(n);
        for (size_t i = 0; i < n; ++i)
            v[i] = amplitude * sinf(step * static_cast<float>(i)) + 0.01f * static_cast<float>(i % 7);
        return v;
    }
}

GPU_TEST(HIP, glue_fusion_softmax_of_a_product)
{
    Shape shape{6, 4, 128};
    auto A = make_shared<op::v0::Parameter>(element::f32, shape);
    auto c = op::v0::Constant::create(element::f32, Shape{}, {0.125f});
    auto scaled = make_shared<op::v1::Multiply>(A, make_shared<op::v0::Broadcast>(c, shape, AxisSet{0, 1, 2}));
    auto f = make_shared<Function>(OutputVector{make_shared<op::v0::Softmax>(scaled, AxisSet{2})}, ParameterVector{A});
    const auto x = wave(shape_size(shape), 9.0f, 0.37f);
    const auto plain = run_glue(f, {x}, false), fused = run_glue(f, {x}, true);
    EXPECT_TRUE(plain.bytes == fused.bytes);
    EXPECT_TRUE(fused.launches < plain.launches);
}

GPU_TEST(HIP, glue_fusion_residual_layer_norm_with_quantize)
{
    // x1 = LayerNorm(a + b) feeds a Quantize (the next projection) and stays live (the next residual)
    Shape shape{9, 768};
    auto a = make_shared<op::v0::Parameter>(element::f32, shape);
    auto b = make_shared<op::v0::Parameter>(element::f32, shape);
    auto g = make_shared<op::v0::Parameter>(element::f32, Shape{768});
    auto be = make_shared<op::v0::Parameter>(element::f32, Shape{768});
    auto sum = make_shared<op::v1::Add>(a, b);
    auto ln = make_shared<op::v0::LayerNorm>(sum, g, be, false, 1, 1e-5);
    auto scale = op::v0::Constant::create(element::f32, Shape{}, {6.0f / 127.0f});
    auto zp = op::v0::Constant::create(element::i8, Shape{}, {-3});
    auto q = make_shared<op::v0::Quantize>(ln, scale, zp, element::i8, AxisSet{}, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
    auto f = make_shared<Function>(OutputVector{ln, q}, ParameterVector{a, b, g, be});
    vector<float> gamma(768), beta(768);
    for (size_t i = 0; i < 768; ++i)
    {
        gamma[i] = 0.8f + 0.0005f * static_cast<float>(i);
        beta[i] = -0.1f + 0.0002f * static_cast<float>(i);
    }
    const vector<vector<float>> args{wave(shape_size(shape), 1.0f, 0.11f), wave(shape_size(shape), 0.3f, 0.53f), gamma, beta};
    const auto plain = run_glue(f, args, false), fused = run_glue(f, args, true);
    EXPECT_TRUE(plain.bytes == fused.bytes);
    EXPECT_TRUE(fused.launches + 2 == plain.launches); // Add and Quantize are gone
    // the quantized copy is not degenerate
    set<uint8_t> codes(fused.bytes[1].begin(), fused.bytes[1].end());
    EXPECT_TRUE(codes.size() > 40);
}

GPU_TEST(HIP, glue_fusion_gelu_with_quantize)
{
    Shape shape{5, 3072};
    auto A = make_shared<op::v0::Parameter>(element::f32, shape);
    auto gelu = make_shared<op::v0::Gelu>(A);
    auto scale = op::v0::Constant::create(element::f32, Shape{}, {0.0175f});
    auto zp = op::v0::Constant::create(element::u8, Shape{}, {16});
    auto q = make_shared<op::v0::Quantize>(gelu, scale, zp, element::u8, AxisSet{}, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
    const auto x = wave(shape_size(shape), 2.5f, 0.071f);
    {
        auto f = make_shared<Function>(OutputVector{q}, ParameterVector{A}); // the Quantize is Gelu's only reader
        const auto plain = run_glue(f, {x}, false), fused = run_glue(f, {x}, true);
        EXPECT_TRUE(plain.bytes == fused.bytes);
        EXPECT_TRUE(fused.launches + 1 == plain.launches);
    }
    {
        auto f = make_shared<Function>(OutputVector{q, gelu}, ParameterVector{A}); // ... and with the f32 result live as well
        const auto plain = run_glue(f, {x}, false), fused = run_glue(f, {x}, true);
        EXPECT_TRUE(plain.bytes == fused.bytes);
        EXPECT_TRUE(fused.launches + 1 == plain.launches);
    }
}

GPU_TEST(HIP, glue_fusion_attention_of_a_batch_of_heads)
{
    // BatchMatMul(Softmax(Multiply(BatchMatMulTranspose(q, k), 1/8)), v) with 128 keys of depth 64: one
    // launch instead of three, the same bits; and the same chain without the Multiply
    const size_t heads = 6, rows = 64, keys = 128, depth = 64;
    for (const bool scaled : {true, false})
    {
        auto q = make_shared<op::v0::Parameter>(element::f32, Shape{heads, rows, depth});
        auto k = make_shared<op::v0::Parameter>(element::f32, Shape{heads, keys, depth});
        auto v = make_shared<op::v0::Parameter>(element::f32, Shape{heads, keys, depth});
        shared_ptr<Node> scores = make_shared<op::v0::BatchMatMulTranspose>(q, k, false, true);
        if (scaled)
            scores = make_shared<op::v1::Multiply>(scores, op::v0::Constant::create(element::f32, Shape{heads, rows, keys}, vector<float>{0.125f}));
        auto probs = make_shared<op::v0::Softmax>(scores, AxisSet{2});
        auto context = make_shared<op::v0::BatchMatMul>(probs, v);
        auto f = make_shared<Function>(NodeVector{context}, ParameterVector{q, k, v});
        const vector<vector<float>> args{wave(heads * rows * depth, 1.5f, 0.37f), wave(heads * keys * depth, 1.2f, 0.11f), wave(heads * keys * depth, 0.8f, 0.23f)};
        const GlueRun fused = run_glue(f, args, true), plain = run_glue(f, args, false);
        EXPECT_TRUE(fused.bytes == plain.bytes);
        EXPECT_EQ(fused.launches, size_t(1));
        EXPECT_EQ(plain.launches, size_t(scaled ? 4 : 3));
    }
    // probabilities with a second reader keep their own launch: nothing is folded past the Multiply
    {
        auto q = make_shared<op::v0::Parameter>(element::f32, Shape{2, 32, depth});
        auto k = make_shared<op::v0::Parameter>(element::f32, Shape{2, keys, depth});
        auto v = make_shared<op::v0::Parameter>(element::f32, Shape{2, keys, depth});
        auto probs = make_shared<op::v0::Softmax>(make_shared<op::v0::BatchMatMulTranspose>(q, k, false, true), AxisSet{2});
        auto context = make_shared<op::v0::BatchMatMul>(probs, v);
        auto f = make_shared<Function>(NodeVector{context, probs}, ParameterVector{q, k, v});
        const vector<vector<float>> args{wave(2 * 32 * depth, 1.0f, 0.3f), wave(2 * keys * depth, 1.0f, 0.7f), wave(2 * keys * depth, 1.0f, 0.9f)};
        const GlueRun fused = run_glue(f, args, true), plain = run_glue(f, args, false);
        EXPECT_TRUE(fused.bytes == plain.bytes);
        EXPECT_EQ(fused.launches, size_t(3));
    }
    // other head shapes stay three launches
    {
        auto q = make_shared<op::v0::Parameter>(element::f32, Shape{3, 16, 8});
        auto k = make_shared<op::v0::Parameter>(element::f32, Shape{3, 16, 8});
        auto probs = make_shared<op::v0::Softmax>(make_shared<op::v0::BatchMatMulTranspose>(q, k, false, true), AxisSet{2});
        auto f = make_shared<Function>(NodeVector{make_shared<op::v0::BatchMatMul>(probs, k)}, ParameterVector{q, k});
        const vector<vector<float>> args{wave(3 * 16 * 8, 1.0f, 0.3f), wave(3 * 16 * 8, 1.0f, 0.7f)};
        const GlueRun fused = run_glue(f, args, true), plain = run_glue(f, args, false);
        EXPECT_TRUE(fused.bytes == plain.bytes);
        EXPECT_EQ(fused.launches, size_t(3));
    }
}

GPU_TEST(HIP, glue_fusion_dot_bias_with_gelu_and_quantize)
{
    // Quantize(Gelu(QuantizedDotBias(Quantize(x), W, b, s) as f32)): Gelu and the Quantize behind it ride
    // in the product's epilogue (512 rows: the tile kernels' own epilogue; 40 rows: through the
    // library's workspace) -- two launches fewer, the same bytes
    for (const size_t rows : {size_t(512), size_t(40)})
    {
        const size_t K = 256, N = 128;
        auto x = make_shared<op::v0::Parameter>(element::f32, Shape{rows, K});
        auto xs = op::v0::Constant::create(element::f32, Shape{}, {0.02f});
        auto xz = op::v0::Constant::create(element::i8, Shape{}, {0});
        auto x8 = make_shared<op::v0::Quantize>(x, xs, xz, element::i8, AxisSet{}, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
        vector<int8_t> w(N * K);
        for (size_t i = 0; i < w.size(); ++i)
            w[i] = static_cast<int8_t>(static_cast<int>((i * 37 + i / K * 11) % 255) - 127);
        vector<int32_t> b(N);
        vector<float> s(N);
        for (size_t i = 0; i < N; ++i)
        {
            b[i] = static_cast<int32_t>(i * 13) - 700;
            s[i] = 0.0002f + 0.000001f * static_cast<float>(i);
        }
        auto W = op::v0::Constant::create(element::i8, Shape{N, K}, w);
        auto B = op::v0::Constant::create(element::i32, Shape{N}, b);
        auto S = op::v0::Constant::create(element::f32, Shape{N}, s);
        auto dot = make_shared<op::v0::QuantizedDotBias>(x8, W, B, S, false, false);
        auto gelu = make_shared<op::v0::Gelu>(dot);
        auto qs = op::v0::Constant::create(element::f32, Shape{}, {0.03f});
        auto qz = op::v0::Constant::create(element::i8, Shape{}, {-3});
        auto q = make_shared<op::v0::Quantize>(gelu, qs, qz, element::i8, AxisSet{}, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
        const auto data = wave(rows * K, 1.8f, 0.013f);
        {
            auto f = make_shared<Function>(OutputVector{q}, ParameterVector{x});
            const auto plain = run_glue(f, {data}, false), fused = run_glue(f, {data}, true);
            EXPECT_TRUE(plain.bytes == fused.bytes);
            EXPECT_EQ(plain.launches, size_t(4)); // Quantize, product, Gelu, Quantize
            EXPECT_EQ(fused.launches, size_t(2)); // Quantize, product with Gelu and Quantize
            size_t distinct[256] = {0}, kinds = 0;
            for (uint8_t v : fused.bytes.at(0))
                kinds += distinct[v]++ == 0;
            EXPECT_TRUE(kinds > 20);
        }
        {
            // the product has a second reader: only the Quantize goes into the Gelu
            auto f = make_shared<Function>(OutputVector{q, dot}, ParameterVector{x});
            const auto plain = run_glue(f, {data}, false), fused = run_glue(f, {data}, true);
            EXPECT_TRUE(plain.bytes == fused.bytes);
            EXPECT_EQ(fused.launches, size_t(3));
        }
    }
}

GPU_TEST(HIP, glue_fusion_dot_bias_gelu_quantize_unpacked_shapes)
{
    // Shapes whose weights the library does not prepack (a reduction of 100 bytes is not a multiple of
    // 16) cannot take the fused entry point: the product keeps its own launch and only the Quantize
    // folds into the Gelu.  A narrow product (8 columns) that is packed takes the workspace route.
    struct Case
    {
        size_t rows, K, N, fused_launches;
    };
    for (const Case c : {Case{48, 100, 24, 3}, Case{300, 100, 128, 3}, Case{64, 64, 8, 2}})
    {
        auto x = make_shared<op::v0::Parameter>(element::f32, Shape{c.rows, c.K});
        auto xs = op::v0::Constant::create(element::f32, Shape{}, {0.02f});
        auto xz = op::v0::Constant::create(element::i8, Shape{}, {0});
        auto x8 = make_shared<op::v0::Quantize>(x, xs, xz, element::i8, AxisSet{}, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
        vector<int8_t> w(c.N * c.K);
        for (size_t i = 0; i < w.size(); ++i)
            w[i] = static_cast<int8_t>(static_cast<int>((i * 29 + i / c.K * 7) % 255) - 127);
        vector<int32_t> b(c.N);
        vector<float> s(c.N);
        for (size_t i = 0; i < c.N; ++i)
        {
            b[i] = static_cast<int32_t>(i * 17) - 300;
            s[i] = 0.0004f + 0.000002f * static_cast<float>(i);
        }
        auto W = op::v0::Constant::create(element::i8, Shape{c.N, c.K}, w);
        auto B = op::v0::Constant::create(element::i32, Shape{c.N}, b);
        auto S = op::v0::Constant::create(element::f32, Shape{c.N}, s);
        auto dot = make_shared<op::v0::QuantizedDotBias>(x8, W, B, S, false, false);
        auto gelu = make_shared<op::v0::Gelu>(dot);
        auto qs = op::v0::Constant::create(element::f32, Shape{}, {0.03f});
        auto qz = op::v0::Constant::create(element::i8, Shape{}, {2});
        auto q = make_shared<op::v0::Quantize>(gelu, qs, qz, element::i8, AxisSet{}, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
        const auto data = wave(c.rows * c.K, 1.8f, 0.013f);
        auto f = make_shared<Function>(OutputVector{q}, ParameterVector{x});
        const auto plain = run_glue(f, {data}, false), fused = run_glue(f, {data}, true);
        EXPECT_TRUE(plain.bytes == fused.bytes);
        EXPECT_EQ(plain.launches, size_t(4));
        EXPECT_EQ(fused.launches, c.fused_launches);
    }
}
