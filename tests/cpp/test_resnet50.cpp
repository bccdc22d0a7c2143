// The synthetic int8 ResNet-50 as an ngraph::Function on backend "HIP": the same network as
// ngraph_amd/resnet50.py (resnet50_graph.hpp), built from Quantize, QuantizedConvolutionBias /
// BiasAdd / BiasSignedAdd, MaxPool, AvgPool, Convert, Reshape, QuantizedDotBias and Dequantize nodes,
// compiled and called like any other function.  Its logits for the seeded image must equal, bit
// for bit, the ones the CPU restatement of the ops computes (tests/golden/resnet50_logits.npz,
// tabled in resnet50_logits.inc).
#include <cstdlib>
#include <cstring>

#include "resnet50_graph.hpp"
#include "test_util.hpp"

using namespace std;
using namespace ngraph;
using resnet50_graph::resnet50;

#include "resnet50_logits.inc"

CPU_TEST(resnet50, graph_shape)
{
    auto f = resnet50(2);
    EXPECT_EQ(f->get_output_shape(0), (Shape{2, 1000}));
    EXPECT_EQ(f->get_output_element_type(0), element::f32);
    EXPECT_EQ(f->get_parameters().at(0)->get_output_element_type(0), element::f32);
    EXPECT_EQ(count_ops_of_type<op::v0::Quantize>(f), 1u);
    EXPECT_EQ(count_ops_of_type<op::v0::Dequantize>(f), 1u);
    EXPECT_EQ(count_ops_of_type<op::v0::QuantizedDotBias>(f), 1u);
    EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolutionBias>(f), 37u); // stem + 16 x 2 + 4 shortcuts
    EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolutionBiasAdd>(f), 12u);
    EXPECT_EQ(count_ops_of_type<op::v0::QuantizedConvolutionBiasSignedAdd>(f), 4u);
}

CPU_TEST(resnet50, seeded_image_is_the_fixture_image)
{
    // the f32 image goes through log / cos / sin of the host's math library: the fixture records the
    // sum of its bit patterns, so a library that rounds one of them differently is named here and not
    // by a logits mismatch
    const auto image = resnet50_graph::synthetic_images(1);
    uint64_t sum = 0;
    for (float v : image)
    {
        uint32_t bits;
        memcpy(&bits, &v, 4);
        sum += bits;
    }
    EXPECT_EQ(sum, kResnet50ImageBitSum);
}

GPU_TEST(HIP, resnet50_function_matches_reference_logits)
{
    auto backend = runtime::Backend::create("HIP");
    auto image = backend->create_tensor(element::f32, Shape{1, 3, 224, 224});
    copy_data(image, resnet50_graph::synthetic_images(1));
    auto logits = backend->create_tensor(element::f32, Shape{1, 1000});
    auto exec = backend->compile(resnet50(1));
    for (int call = 0; call < 4; ++call) // eager, captured, replayed twice
    {
        exec->call_with_validate({logits}, {image});
        auto got = read_vector<float>(logits);
        size_t same = 0;
        for (size_t i = 0; i < 1000; ++i)
        {
            uint32_t bits;
            memcpy(&bits, &got[i], 4);
            same += bits == kResnet50LogitBits[i];
        }
        EXPECT_EQ(same, 1000u);
    }
}
