// The plugin boundary, written after the reference's test/backend/api.in.cpp:31-100,
// test/backend/validate_call.in.cpp:31-131, test/backend/unhandled_op.in.cpp:25-66 and
// test/backend_api.cpp:27-81, against backend "HIP".
#include <algorithm>

#include "test_util.hpp"

using namespace std;
using namespace ngraph;

GPU_TEST(HIP, create_tensor_1)
{
    Shape shape{2, 2};
    auto A = make_shared<op::v0::Parameter>(element::f32, shape);
    auto B = make_shared<op::v0::Parameter>(element::f32, shape);
    auto f = make_shared<Function>(make_shared<op::v1::Add>(A, B), ParameterVector{A, B});
    auto backend = runtime::Backend::create("HIP");
    vector<float> av = {1, 2, 3, 4};
    vector<float> bv = {5, 6, 7, 8};
    auto a = backend->create_tensor(element::f32, shape);
    auto b = backend->create_tensor(element::f32, shape);
    copy_data(a, av);
    copy_data(b, bv);
    auto result = backend->create_tensor(element::f32, shape);
    auto handle = backend->compile(f);
    handle->call_with_validate({result}, {a, b});
    EXPECT_VEC_EQ((vector<float>{6, 8, 10, 12}), read_vector<float>(result));
}

GPU_TEST(HIP, tensor_copy_from)
{
    Shape shape{2, 2};
    auto backend = runtime::Backend::create("HIP");
    vector<float> av = {1, 2, 3, 4};
    vector<float> bv = {5, 6, 7, 8};
    auto a = backend->create_tensor(element::f32, shape);
    auto b = backend->create_tensor(element::f32, shape);
    copy_data(a, av);
    copy_data(b, bv);
    a->copy_from(*b);
    EXPECT_VEC_EQ(bv, read_vector<float>(a));
    // a host tensor as the source goes through the default bounce
    runtime::HostTensor h(element::f32, shape);
    h.write(av.data(), av.size() * sizeof(float));
    b->copy_from(h);
    EXPECT_VEC_EQ(av, read_vector<float>(b));
}

GPU_TEST(HIP, get_parameters_and_results)
{
    Shape shape{2, 2};
    auto A = make_shared<op::v0::Parameter>(element::f32, shape);
    auto B = make_shared<op::v0::Parameter>(element::f32, shape);
    auto C = make_shared<op::v0::Parameter>(element::f32, shape);
    auto f = make_shared<Function>((A + B) * C, ParameterVector{A, B, C});
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor(element::f32, shape);
    auto b = backend->create_tensor(element::f32, shape);
    auto c = backend->create_tensor(element::f32, shape);
    auto result = backend->create_tensor(element::f32, shape);
    copy_data(a, vector<float>{1, 2, 3, 4});
    copy_data(b, vector<float>{5, 6, 7, 8});
    copy_data(c, vector<float>{9, 10, 11, 12});
    auto handle = backend->compile(f);
    EXPECT_EQ(handle->get_parameters().size(), 3u);
    EXPECT_EQ(handle->get_results().size(), 1u);
    handle->call_with_validate({result}, {a, b, c});
    EXPECT_VEC_EQ((vector<float>{54, 80, 110, 144}), read_vector<float>(result));
    // compile must leave the caller's function alone and cache by function
    EXPECT_EQ(f->get_ordered_ops().size(), 6u);
    EXPECT_TRUE(backend->compile(f) == handle);
}

namespace
{
    struct AddFixture
    {
        shared_ptr<Function> f;
        shared_ptr<runtime::Backend> backend = runtime::Backend::create("HIP");
        AddFixture()
        {
            Shape shape{2, 2};
            auto A = make_shared<op::v0::Parameter>(element::f32, shape);
            auto B = make_shared<op::v0::Parameter>(element::f32, shape);
            f = make_shared<Function>(make_shared<op::v1::Add>(A, B), ParameterVector{A, B});
        }
    };
}

GPU_TEST(HIP, validate_call_input_count)
{
    AddFixture x;
    auto a = x.backend->create_tensor(element::f32, Shape{2, 2});
    auto c = x.backend->create_tensor(element::f32, Shape{2, 2});
    EXPECT_THROW(auto handle = x.backend->compile(x.f); handle->call_with_validate({c}, {a}), std::runtime_error);
}

GPU_TEST(HIP, validate_call_input_type)
{
    AddFixture x;
    auto a = x.backend->create_tensor(element::i32, Shape{2, 2});
    auto b = x.backend->create_tensor(element::f32, Shape{2, 2});
    auto c = x.backend->create_tensor(element::f32, Shape{2, 2});
    EXPECT_THROW(auto handle = x.backend->compile(x.f); handle->call_with_validate({c}, {a, b}), std::runtime_error);
}

GPU_TEST(HIP, validate_call_input_shape)
{
    AddFixture x;
    auto a = x.backend->create_tensor(element::f32, Shape{2, 3});
    auto b = x.backend->create_tensor(element::f32, Shape{2, 2});
    auto c = x.backend->create_tensor(element::f32, Shape{2, 2});
    EXPECT_THROW(auto handle = x.backend->compile(x.f); handle->call_with_validate({c}, {a, b}), std::runtime_error);
}

GPU_TEST(HIP, validate_call_output_count)
{
    AddFixture x;
    auto a = x.backend->create_tensor(element::f32, Shape{2, 2});
    auto b = x.backend->create_tensor(element::f32, Shape{2, 2});
    auto c = x.backend->create_tensor(element::f32, Shape{2, 2});
    auto d = x.backend->create_tensor(element::f32, Shape{2, 2});
    EXPECT_THROW(auto handle = x.backend->compile(x.f); handle->call_with_validate({c, d}, {a, b}), std::runtime_error);
}

GPU_TEST(HIP, validate_call_output_type)
{
    AddFixture x;
    auto a = x.backend->create_tensor(element::i32, Shape{2, 2});
    auto b = x.backend->create_tensor(element::f32, Shape{2, 2});
    auto c = x.backend->create_tensor(element::f32, Shape{2, 2});
    EXPECT_THROW(auto handle = x.backend->compile(x.f); handle->call_with_validate({a}, {b, c}), std::runtime_error);
}

GPU_TEST(HIP, validate_call_output_shape)
{
    AddFixture x;
    auto a = x.backend->create_tensor(element::f32, Shape{2, 3});
    auto b = x.backend->create_tensor(element::f32, Shape{2, 2});
    auto c = x.backend->create_tensor(element::f32, Shape{2, 2});
    EXPECT_THROW(auto handle = x.backend->compile(x.f); handle->call_with_validate({a}, {c, b}), std::runtime_error);
}

namespace
{
    class UnhandledOp : public ngraph::op::Op
    {
    public:
        UnhandledOp(const Output<Node>& arg) : Op({arg}) { constructor_validate_and_infer_types(); }
        shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override { return make_shared<UnhandledOp>(new_args[0]); }
        static constexpr NodeTypeInfo type_info{"UnhandledOp", 0};
        const NodeTypeInfo& get_type_info() const override { return type_info; }

    protected:
        void validate_and_infer_types() override { set_output_type(0, get_input_element_type(0), get_input_partial_shape(0)); }
    };
    constexpr NodeTypeInfo UnhandledOp::type_info;
}

GPU_TEST(HIP, unhandled_op)
{
    Shape shape{2, 2};
    auto A = make_shared<op::v0::Parameter>(element::f32, shape);
    auto unhandled = make_shared<UnhandledOp>(A);
    auto f = make_shared<Function>(unhandled, ParameterVector{A});
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor<float>(shape);
    auto result = backend->create_tensor<float>(shape);
    EXPECT_THROW(auto handle = backend->compile(f); handle->call_with_validate({result}, {a}), unsupported_op);
    EXPECT_FALSE(backend->is_supported(*unhandled));
    EXPECT_TRUE(backend->is_supported(*A));
}

GPU_TEST(HIP, tensor_partial_and_null_transfers_throw)
{
    auto backend = runtime::Backend::create("HIP");
    auto a = backend->create_tensor(element::f32, Shape{4});
    vector<float> v(4, 1.0f);
    EXPECT_THROW(a->write(v.data(), 8), std::out_of_range);
    EXPECT_THROW(a->read(v.data(), 8), std::out_of_range);
    EXPECT_THROW(a->write(nullptr, 16), std::runtime_error);
}

GPU_TEST(HIP, bad_device_ordinal)
{
    EXPECT_THROW(runtime::Backend::create("HIP:99"), std::runtime_error);
    EXPECT_THROW(runtime::Backend::create("HIP:zero"), std::runtime_error);
    EXPECT_NO_THROW(runtime::Backend::create("HIP:0"));
}

GPU_TEST(HIP, executable_can_create_tensors_and_performance_data)
{
    auto backend = runtime::Backend::create("HIP");
    EXPECT_TRUE(backend->executable_can_create_tensors());
    Shape shape{8};
    auto A = make_shared<op::v0::Parameter>(element::f32, shape);
    auto B = make_shared<op::v0::Parameter>(element::f32, shape);
    auto f = make_shared<Function>((A + B) * A, ParameterVector{A, B});
    auto exec = backend->compile(f, true);
    auto a = exec->create_input_tensor(0);
    auto b = exec->create_input_tensor(1);
    auto r = exec->create_output_tensor(0);
    copy_data(a, vector<float>(8, 2.0f));
    copy_data(b, vector<float>(8, 3.0f));
    exec->call_with_validate({r}, {a, b});
    exec->call_with_validate({r}, {a, b});
    EXPECT_VEC_EQ(vector<float>(8, 10.0f), read_vector<float>(r));
    auto perf = exec->get_performance_data();
    EXPECT_EQ(perf.size(), 2u);
    for (const auto& p : perf)
        EXPECT_EQ(p.call_count(), 2u);
}

// ---- without a GPU ---------------------------------------------------------------------------

CPU_TEST(backend_api, registered_devices)
{
    vector<string> devices = runtime::Backend::get_registered_devices();
    EXPECT_TRUE(find(devices.begin(), devices.end(), "HIP") != devices.end());
}

CPU_TEST(backend_api, invalid_name)
{
    EXPECT_THROW(runtime::Backend::create("COMPLETELY-BOGUS-NAME"), std::runtime_error);
}

CPU_TEST(backend_api, host_tensor)
{
    runtime::HostTensor t(element::i8, Shape{2, 3});
    vector<int8_t> v{1, 2, 3, 4, 5, 6}, r(6);
    t.write(v.data(), 6);
    t.read(r.data(), 6);
    EXPECT_VEC_EQ(v, r);
    EXPECT_THROW(t.write(v.data(), 5), std::out_of_range);
    EXPECT_THROW(t.read(nullptr, 6), std::runtime_error);
    EXPECT_EQ(t.get_size_in_bytes(), 6u);
}
