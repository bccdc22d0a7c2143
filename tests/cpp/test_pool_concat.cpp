// MaxPool / AvgPool / Concat through backend "HIP", with the values of the reference's
// test/backend/pool.in.cpp:64-154,286-341,810-872 and test/backend/concat.in.cpp (matrix / vector
// cases), plus a small quantized block (convolution -> max pool -> concat) the way int8 networks
// chain them; type propagation after test/type_prop/concat.cpp.
#include "test_util.hpp"

using namespace std;
using namespace ngraph;

namespace
{
    template <typename T, typename OP, typename... Extra>
    vector<T> run_pool(const element::Type& et, const Shape& shape_a, const Shape& shape_r, const vector<T>& data, const Shape& window,
                       const Strides& strides, const Shape& pb, const Shape& pa, Extra... extra)
    {
        auto A = make_shared<op::v0::Parameter>(et, shape_a);
        auto P = make_shared<OP>(A, window, strides, pb, pa, extra...);
        auto f = make_shared<Function>(OutputVector{P}, ParameterVector{A});
        auto backend = runtime::Backend::create("HIP");
        auto a = backend->create_tensor(et, shape_a);
        copy_data(a, data);
        auto result = backend->create_tensor(et, shape_r);
        auto handle = backend->compile(f);
        handle->call_with_validate({result}, {a});
        return read_vector<T>(result);
    }
}

GPU_TEST(HIP, max_pool_uint8)
{
    auto r = run_pool<uint8_t, op::v0::MaxPool>(element::u8, Shape{1, 1, 3, 5}, Shape{1, 1, 2, 3}, {0, 1, 0, 2, 1, 0, 3, 2, 0, 0, 2, 0, 0, 0, 1},
                                                Shape{2, 3}, Strides{1, 1}, Shape{0, 0}, Shape{0, 0});
    EXPECT_VEC_EQ((vector<uint8_t>{3, 3, 2, 3, 3, 2}), r);
}

GPU_TEST(HIP, max_pool_int8)
{
    auto r = run_pool<int8_t, op::v0::MaxPool>(element::i8, Shape{1, 1, 3, 5}, Shape{1, 1, 2, 3}, {0, 1, 0, -2, 1, 0, -3, 2, 0, 0, 2, 0, 0, 0, 1},
                                               Shape{2, 3}, Strides{1, 1}, Shape{0, 0}, Shape{0, 0});
    EXPECT_VEC_EQ((vector<int8_t>{2, 2, 2, 2, 2, 2}), r);
}

GPU_TEST(HIP, avg_pool_uint8)
{
    auto r = run_pool<uint8_t, op::v0::AvgPool>(element::u8, Shape{1, 1, 3, 5}, Shape{1, 1, 2, 3}, {0, 1, 0, 2, 1, 0, 3, 2, 0, 0, 2, 0, 0, 0, 1},
                                                Shape{2, 3}, Strides{1, 1}, Shape{0, 0}, Shape{0, 0}, false);
    EXPECT_VEC_EQ((vector<uint8_t>{1, 1, 1, 1, 1, 0}), r);
}

GPU_TEST(HIP, avg_pool_int8)
{
    auto r = run_pool<int8_t, op::v0::AvgPool>(element::i8, Shape{1, 1, 3, 5}, Shape{1, 1, 2, 3}, {10, 1, 0, -2, 1, 0, -3, 4, 0, 0, 2, 0, 0, 0, 1},
                                               Shape{2, 3}, Strides{1, 1}, Shape{0, 0}, Shape{0, 0}, false);
    EXPECT_VEC_EQ((vector<int8_t>{2, 0, 0, 0, 0, 1}), r);
}

GPU_TEST(HIP, max_pool_2d_2channel_2image_asym_pad)
{
    vector<float> x{0, 1, 0, 2, 0, 3, 2, 0, 2, 0, 0, 0, 0, 2, 1, 0, 0, 0, 0, 2, 0, 2, 3, 0, 2, 0, 1, 0, 2, 0, 0, 0,
                    0, 2, 1, 1, 0, 0, 2, 0, 0, 0, 1, 2, 0, 0, 0, 0, 2, 1, 0, 0, 0, 2, 0, 0, 1, 1, 2, 0, 1, 0, 0, 0};
    auto r = run_pool<float, op::v0::MaxPool>(element::f32, Shape{2, 2, 4, 4}, Shape{2, 2, 2, 2}, x, Shape{3, 3}, Strides{2, 2}, Shape{0, 0}, Shape{1, 1});
    EXPECT_VEC_EQ((vector<float>{3, 2, 2, 1, 3, 3, 2, 1, 2, 2, 1, 2, 2, 2, 2, 2}), r);
}

GPU_TEST(HIP, avg_pool_2d_1channel_1image_padded)
{
    vector<float> x{0, 1, 0, 0, 3, 2, 2, 0, 0};
    auto excl = run_pool<float, op::v0::AvgPool>(element::f32, Shape{1, 1, 3, 3}, Shape{1, 1, 4, 4}, x, Shape{2, 2}, Strides{1, 1}, Shape{1, 1}, Shape{1, 1}, false);
    EXPECT_VEC_EQ((vector<float>{0.0f, 0.5f, 0.5f, 0.0f, 0.0f, 1.0f, 1.5f, 1.0f, 1.0f, 1.25f, 1.25f, 1.0f, 2.0f, 1.0f, 0.0f, 0.0f}), excl);
    auto incl = run_pool<float, op::v0::AvgPool>(element::f32, Shape{1, 1, 3, 3}, Shape{1, 1, 4, 4}, x, Shape{2, 2}, Strides{1, 1}, Shape{1, 1}, Shape{1, 1}, true);
    EXPECT_VEC_EQ((vector<float>{0.0f, 0.25f, 0.25f, 0.0f, 0.0f, 1.0f, 1.5f, 0.5f, 0.5f, 1.25f, 1.25f, 0.5f, 0.5f, 0.5f, 0.0f, 0.0f}), incl);
}

GPU_TEST(HIP, concat_matrix_colwise_rowwise)
{
    auto backend = runtime::Backend::create("HIP");
    {
        Shape sa{2, 2}, sb{2, 3}, sc{2, 3}, sr{2, 8};
        auto A = make_shared<op::v0::Parameter>(element::f32, sa);
        auto B = make_shared<op::v0::Parameter>(element::f32, sb);
        auto C = make_shared<op::v0::Parameter>(element::f32, sc);
        auto f = make_shared<Function>(OutputVector{make_shared<op::v0::Concat>(OutputVector{A, B, C}, 1)}, ParameterVector{A, B, C});
        auto a = backend->create_tensor(element::f32, sa);
        copy_data(a, vector<float>{2, 4, 8, 16});
        auto b = backend->create_tensor(element::f32, sb);
        copy_data(b, vector<float>{1, 2, 4, 8, 16, 32});
        auto c = backend->create_tensor(element::f32, sc);
        copy_data(c, vector<float>{2, 3, 5, 7, 11, 13});
        auto result = backend->create_tensor(element::f32, sr);
        backend->compile(f)->call_with_validate({result}, {a, b, c});
        EXPECT_VEC_EQ((vector<float>{2, 4, 1, 2, 4, 2, 3, 5, 8, 16, 8, 16, 32, 7, 11, 13}), read_vector<float>(result));
    }
    {
        Shape sa{2, 2}, sb{3, 2}, sc{3, 2}, sr{8, 2};
        auto A = make_shared<op::v0::Parameter>(element::u8, sa);
        auto B = make_shared<op::v0::Parameter>(element::u8, sb);
        auto C = make_shared<op::v0::Parameter>(element::u8, sc);
        auto f = make_shared<Function>(OutputVector{make_shared<op::v0::Concat>(OutputVector{A, B, C}, -2)}, ParameterVector{A, B, C});
        auto a = backend->create_tensor(element::u8, sa);
        copy_data(a, vector<uint8_t>{2, 4, 8, 16});
        auto b = backend->create_tensor(element::u8, sb);
        copy_data(b, vector<uint8_t>{1, 2, 4, 8, 16, 32});
        auto c = backend->create_tensor(element::u8, sc);
        copy_data(c, vector<uint8_t>{2, 3, 5, 7, 11, 13});
        auto result = backend->create_tensor(element::u8, sr);
        backend->compile(f)->call_with_validate({result}, {a, b, c});
        EXPECT_VEC_EQ((vector<uint8_t>{2, 4, 8, 16, 1, 2, 4, 8, 16, 32, 2, 3, 5, 7, 11, 13}), read_vector<uint8_t>(result));
    }
}

// convolution -> max pool, twice, joined on the channel axis: the pool and the concat work on the
// convolution's u8 output without leaving the device; max pooling commutes with the two separate
// branches, so the joined tensor must equal the two pooled halves
GPU_TEST(HIP, quantized_block_conv_pool_concat)
{
    Shape shape_a{1, 1, 4, 4}, shape_b{2, 1, 1, 1};
    auto A = make_shared<op::v0::Parameter>(element::u8, shape_a);
    auto B1 = op::v0::Constant::create(element::i8, shape_b, {1, 2});
    auto B2 = op::v0::Constant::create(element::i8, shape_b, {3, -1});
    auto one = op::v0::Constant::create(element::f32, Shape{}, {1.0f});
    auto zu = op::v0::Constant::create(element::u8, Shape{}, {0});
    auto zi = op::v0::Constant::create(element::i8, Shape{}, {0});
    auto conv = [&](const shared_ptr<Node>& w) {
        return make_shared<op::v0::QuantizedConvolution>(A, w, Strides{1, 1}, Strides{1, 1}, CoordinateDiff{0, 0}, CoordinateDiff{0, 0}, Strides{1, 1},
                                                         one, zu, one, zi, one, zu, element::u8);
    };
    auto p1 = make_shared<op::v0::MaxPool>(conv(B1), Shape{2, 2}, Strides{2, 2}, Shape{0, 0}, Shape{0, 0});
    auto p2 = make_shared<op::v0::MaxPool>(conv(B2), Shape{2, 2}, Strides{2, 2}, Shape{0, 0}, Shape{0, 0});
    auto cat = make_shared<op::v0::Concat>(OutputVector{p1, p2}, 1);
    auto f = make_shared<Function>(OutputVector{cat}, ParameterVector{A});
    EXPECT_EQ(cat->get_output_shape(0), (Shape{1, 4, 2, 2}));
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor(element::u8, shape_a);
    copy_data(a, vector<uint8_t>{1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16});
    auto result = backend->create_tensor(element::u8, Shape{1, 4, 2, 2});
    backend->compile(f)->call_with_validate({result}, {a});
    // pooled input is {6, 8, 14, 16} for the channels x1, x2, x3; the x(-1) channel wraps into u8 the way
    // the reference kernel's static_cast does (src/ngraph/runtime/reference/convolution.hpp:255-257), so
    // its window maxima are those of {255, 254, 251, 250}, {253, ...}, {247, ...}, {245, ...}
    EXPECT_VEC_EQ((vector<uint8_t>{6, 8, 14, 16, 12, 16, 28, 32, 18, 24, 42, 48, 255, 253, 247, 245}), read_vector<uint8_t>(result));
}

CPU_TEST(type_prop, concat_and_pool_shapes)
{
    auto A = make_shared<op::v0::Parameter>(element::u8, Shape{2, 3, 4});
    auto B = make_shared<op::v0::Parameter>(element::u8, Shape{2, 7, 4});
    auto C = make_shared<op::v0::Parameter>(element::u8, Shape{2, 2, 4});
    auto cc = make_shared<op::v0::Concat>(OutputVector{A, B, C}, 1);
    EXPECT_EQ(cc->get_output_shape(0), (Shape{2, 12, 4}));
    EXPECT_EQ(cc->get_output_element_type(0), element::u8);
    EXPECT_EQ(make_shared<op::v0::Concat>(OutputVector{A, B, C}, -2)->get_concatenation_axis(), 1);
    auto D = make_shared<op::v0::Parameter>(element::u8, Shape{2, 3, 5});
    EXPECT_THROW(make_shared<op::v0::Concat>(OutputVector{A, D}, 1), NodeValidationFailure);
    auto E = make_shared<op::v0::Parameter>(element::i8, Shape{2, 3, 4});
    EXPECT_THROW(make_shared<op::v0::Concat>(OutputVector{A, E}, 1), NodeValidationFailure);
    EXPECT_THROW(make_shared<op::v0::Concat>(OutputVector{A, B}, 3), NodeValidationFailure);
    auto X = make_shared<op::v0::Parameter>(element::u8, Shape{8, 64, 112, 112});
    auto mp = make_shared<op::v0::MaxPool>(X, Shape{3, 3}, Strides{2, 2}, Shape{1, 1}, Shape{1, 1});
    EXPECT_EQ(mp->get_output_shape(0), (Shape{8, 64, 56, 56}));
}

// op::v1::Divide on integers: floor division unless the op says otherwise (values of the
// reference's test/backend/divide.in.cpp:69-133)
namespace
{
    vector<int32_t> run_divide(const vector<int32_t>& x, const vector<int32_t>& y, bool set_flag, bool pythondiv)
    {
        Shape shape{2, 2};
        auto A = make_shared<op::v0::Parameter>(element::i32, shape);
        auto B = make_shared<op::v0::Parameter>(element::i32, shape);
        auto div = set_flag ? make_shared<op::v1::Divide>(A, B, pythondiv) : make_shared<op::v1::Divide>(A, B);
        auto f = make_shared<Function>(OutputVector{div}, ParameterVector{A, B});
        auto backend = runtime::Backend::create("HIP");
        auto a = backend->create_tensor(element::i32, shape);
        copy_data(a, x);
        auto b = backend->create_tensor(element::i32, shape);
        copy_data(b, y);
        auto result = backend->create_tensor(element::i32, shape);
        backend->compile(f)->call_with_validate({result}, {a, b});
        return read_vector<int32_t>(result);
    }
}

GPU_TEST(HIP, divide_int32)
{
    EXPECT_VEC_EQ((vector<int32_t>{536871072, 214748365, 2, 2}), run_divide({0x40000140, 0x40000001, 8, 16}, {2, 5, 4, 8}, false, true));
}

GPU_TEST(HIP, divide_cpp_rounding_int32)
{
    EXPECT_VEC_EQ((vector<int32_t>{3, -3, -3, 3}), run_divide({-10, -10, 10, 10}, {-3, 3, -3, 3}, true, false));
}

GPU_TEST(HIP, divide_python_rounding_int32)
{
    EXPECT_VEC_EQ((vector<int32_t>{3, -4, -4, 3}), run_divide({-10, -10, 10, 10}, {-3, 3, -3, 3}, false, true));
}
