// op::v0::Slice of the host subset: shape deduction and its errors as test/type_prop/slice.cpp:24-277
// of the nGraph tree has them, the backend "HIP" against the vectors of test/backend/slice.in.cpp,
// and a trip through the serializer.
#include "ngraph/serializer.hpp"
#include "test_util.hpp"

using namespace std;
using namespace ngraph;

namespace
{
    string what_of(const function<void()>& fn)
    {
        try
        {
            fn();
        }
        catch (const NodeValidationFailure& e)
        {
            return e.what();
        }
        return "";
    }
}

CPU_TEST(type_prop, slice_deduces_shapes)
{
    auto v = make_shared<op::v0::Parameter>(element::f32, Shape{6});
    auto m = make_shared<op::v0::Parameter>(element::f32, Shape{6, 8});
    EXPECT_EQ(make_shared<op::v0::Slice>(v, Coordinate{2}, Coordinate{5})->get_output_shape(0), (Shape{3}));
    EXPECT_EQ(make_shared<op::v0::Slice>(m, Coordinate{2, 1}, Coordinate{5, 7})->get_output_shape(0), (Shape{3, 6}));
    EXPECT_EQ(make_shared<op::v0::Slice>(m, Coordinate{2, 1}, Coordinate{5, 7}, Strides{3, 2})->get_output_shape(0), (Shape{1, 3}));
    EXPECT_EQ(make_shared<op::v0::Slice>(m, Coordinate{2, 1}, Coordinate{5, 8}, Strides{3, 2})->get_output_shape(0), (Shape{1, 4})); // uneven: rounded up
    EXPECT_EQ(make_shared<op::v0::Slice>(v, Coordinate{0}, Coordinate{6})->get_output_shape(0), (Shape{6}));
    EXPECT_EQ(make_shared<op::v0::Slice>(m, Coordinate{0, 0}, Coordinate{6, 8})->get_output_shape(0), (Shape{6, 8}));
    EXPECT_EQ(make_shared<op::v0::Slice>(m, Coordinate{0, 0}, Coordinate{6, 0})->get_output_shape(0), (Shape{6, 0}));
    EXPECT_EQ(make_shared<op::v0::Slice>(m, Coordinate{0, 0}, Coordinate{0, 0})->get_output_shape(0), (Shape{0, 0}));
    auto i8 = make_shared<op::v0::Parameter>(element::i8, Shape{2, 3});
    EXPECT_EQ(make_shared<op::v0::Slice>(i8, Coordinate{0, 1}, Coordinate{2, 3})->get_output_element_type(0), element::i8);
    // the default strides are ones
    EXPECT_EQ(make_shared<op::v0::Slice>(m, Coordinate{0, 0}, Coordinate{6, 8})->get_strides(), (Strides{1, 1}));
}

CPU_TEST(type_prop, slice_rejects_what_the_reference_rejects)
{
    auto v = make_shared<op::v0::Parameter>(element::f32, Shape{6});
    auto m = make_shared<op::v0::Parameter>(element::f32, Shape{6, 8});
    EXPECT_TRUE(what_of([&] { make_shared<op::v0::Slice>(v, Coordinate{0}, Coordinate{7}, Strides{1, 2}); }).find("Ranks of lower bounds (") != string::npos);
    EXPECT_TRUE(what_of([&] { make_shared<op::v0::Slice>(v, Coordinate{0}, Coordinate{7}); }).find("Upper bound for slice at axis 0 is out of range (upper bounds: ") != string::npos);
    EXPECT_TRUE(what_of([&] { make_shared<op::v0::Slice>(m, Coordinate{0, 0}, Coordinate{6, 9}); }).find("Upper bound for slice at axis 1 is out of range") != string::npos);
    EXPECT_TRUE(what_of([&] { make_shared<op::v0::Slice>(v, Coordinate{3}, Coordinate{2}); }).find("Lower bound for slice is greater than upper bound at axis 0 (lower bounds: ") != string::npos);
    EXPECT_TRUE(what_of([&] { make_shared<op::v0::Slice>(m, Coordinate{0, 5}, Coordinate{6, 4}); }).find("Lower bound for slice is greater than upper bound at axis 1") != string::npos);
    EXPECT_TRUE(what_of([&] { make_shared<op::v0::Slice>(m, Coordinate{0}, Coordinate{5, 5}); }).find("Ranks of lower bounds") != string::npos);
    EXPECT_TRUE(what_of([&] { make_shared<op::v0::Slice>(m, Coordinate{0, 0}, Coordinate{5}); }).find("Ranks of lower bounds") != string::npos);
    EXPECT_TRUE(what_of([&] { make_shared<op::v0::Slice>(m, Coordinate{0, 0, 0}, Coordinate{5, 5, 5}); }).find("Input rank does not match the rank of the lower bounds") != string::npos);
    EXPECT_TRUE(what_of([&] { make_shared<op::v0::Slice>(m, Coordinate{0, 0}, Coordinate{5, 5}, Strides{1, 0}); }).find("Stride for slice is zero at axis 1 (strides: ") != string::npos);
}

CPU_TEST(serializer, slice_round_trip)
{
    auto a = make_shared<op::v0::Parameter>(element::f32, Shape{4, 4, 4});
    auto s = make_shared<op::v0::Slice>(a, Coordinate{0, 1, 0}, Coordinate{4, 3, 4}, Strides{2, 1, 3});
    auto f = make_shared<Function>(NodeVector{s}, ParameterVector{a});
    const string js = serialize(f, 0);
    EXPECT_TRUE(js.find("\"lower_bounds\":[0,1,0]") != string::npos);
    EXPECT_TRUE(js.find("\"upper_bounds\":[4,3,4]") != string::npos);
    EXPECT_TRUE(js.find("\"strides\":[2,1,3]") != string::npos);
    auto g = deserialize(js);
    shared_ptr<op::v0::Slice> back;
    for (const auto& n : g->get_ordered_ops())
        if (auto t = as_type_ptr<op::v0::Slice>(n))
            back = t;
    EXPECT_TRUE(back != nullptr);
    EXPECT_EQ(back->get_lower_bounds(), (Coordinate{0, 1, 0}));
    EXPECT_EQ(back->get_upper_bounds(), (Coordinate{4, 3, 4}));
    EXPECT_EQ(back->get_strides(), (Strides{2, 1, 3}));
    EXPECT_EQ(back->get_output_shape(0), (Shape{2, 2, 2}));
}

// test/backend/slice.in.cpp:30-92,223-378
GPU_TEST(HIP, slice_vectors)
{
    auto backend = runtime::Backend::create("HIP");
    auto run = [&](const Shape& shape, const Coordinate& lower, const Coordinate& upper, const Strides& strides, const vector<float>& data) {
        auto A = make_shared<op::v0::Parameter>(element::f32, shape);
        auto r = strides.empty() ? make_shared<op::v0::Slice>(A, lower, upper) : make_shared<op::v0::Slice>(A, lower, upper, strides);
        auto f = make_shared<Function>(r, ParameterVector{A});
        auto a = backend->create_tensor(element::f32, shape);
        copy_data(a, data);
        auto result = backend->create_tensor(element::f32, r->get_output_shape(0));
        backend->compile(f)->call_with_validate({result}, {a});
        return read_vector<float>(result);
    };
    vector<float> ramp16(16), ramp64(64);
    for (size_t i = 0; i < 16; ++i)
        ramp16[i] = static_cast<float>(i + 1);
    for (size_t i = 0; i < 64; ++i)
        ramp64[i] = static_cast<float>(i);
    EXPECT_VEC_EQ((vector<float>{2, 3, 6, 7, 10, 11}), run(Shape{4, 4}, Coordinate{0, 1}, Coordinate{3, 3}, Strides{}, ramp16));
    vector<float> zero_based(ramp16);
    for (auto& x : zero_based)
        x -= 1.0f;
    EXPECT_VEC_EQ((vector<float>{2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13}), run(Shape{16}, Coordinate{2}, Coordinate{14}, Strides{}, zero_based));
    EXPECT_VEC_EQ((vector<float>{4, 7, 12, 15}), run(Shape{4, 4}, Coordinate{1, 0}, Coordinate{4, 4}, Strides{2, 3}, zero_based));
    EXPECT_VEC_EQ((vector<float>{21, 22, 25, 26, 37, 38, 41, 42}), run(Shape{4, 4, 4}, Coordinate{1, 1, 1}, Coordinate{3, 3, 3}, Strides{}, ramp64));
    EXPECT_VEC_EQ((vector<float>{0, 2, 8, 10, 32, 34, 40, 42}), run(Shape{4, 4, 4}, Coordinate{0, 0, 0}, Coordinate{4, 4, 4}, Strides{2, 2, 2}, ramp64));
    EXPECT_VEC_EQ((vector<float>{0, 3, 8, 11, 32, 35, 40, 43}), run(Shape{4, 4, 4}, Coordinate{0, 0, 0}, Coordinate{4, 4, 4}, Strides{2, 2, 3}, ramp64));
    // a lower bound at the end of its axis: an empty result
    EXPECT_VEC_EQ((vector<float>{}), run(Shape{20, 10, 5}, Coordinate{0, 10, 0}, Coordinate{20, 10, 5}, Strides{1, 1, 1}, vector<float>(20 * 10 * 5, 222.0f)));
    // a scalar slices to itself (followed by Abs, as in the reference's test)
    {
        auto A = make_shared<op::v0::Parameter>(element::f32, Shape{});
        auto r = make_shared<op::v0::Slice>(A, Coordinate{}, Coordinate{});
        auto f = make_shared<Function>(make_shared<op::v0::Abs>(r), ParameterVector{A});
        auto a = backend->create_tensor(element::f32, Shape{});
        copy_data(a, vector<float>{312});
        auto result = backend->create_tensor(element::f32, Shape{});
        backend->compile(f)->call_with_validate({result}, {a});
        EXPECT_VEC_EQ((vector<float>{312}), read_vector<float>(result));
    }
}
