// Builders of the quantized ops: min/max ranges -> scale sub-graphs -> op.
// Algebra restated from src/ngraph/builder/quantization_utils.cpp:33-174,
// quantize_builder.cpp:27-57, dequantize_builder.cpp:27-56, quantized_conv_builder.cpp:28-333 and
// quantized_dot_builder.cpp:28-118 of the nGraph tree.
#include <cmath>
#include <limits>

#include "ngraph/builder.hpp"

using namespace std;

namespace ngraph
{
    namespace builder
    {
        namespace quantization_utils
        {
            static void same_type_and_shape(const char* who, std::initializer_list<Output<Node>> v)
            {
                const Output<Node>& first = *v.begin();
                for (const auto& o : v)
                {
                    if (o.get_element_type() != first.get_element_type())
                        throw ngraph_error(string(who) + ": min and max must have same type");
                    if (o.get_shape() != first.get_shape())
                        throw ngraph_error(string(who) + ": min and max must have same shape");
                }
            }

            shared_ptr<Node> max_abs(const Output<Node>& a, const Output<Node>& b)
            {
                return make_shared<op::v1::Maximum>(make_shared<op::v0::Abs>(a), make_shared<op::v0::Abs>(b));
            }

            shared_ptr<Node> get_scale(const Output<Node>& input_min_range,
                                       const Output<Node>& input_max_range,
                                       const element::Type& quant_type,
                                       bool bump_by_eps)
            {
                same_type_and_shape("get_scale", {input_min_range, input_max_range});
                const auto type = input_min_range.get_element_type();
                const auto shape = input_min_range.get_shape();
                Output<Node> lo = input_min_range, hi = input_max_range;
                if (bump_by_eps)
                {
                    // the quantized range must contain 0 and be at least max(1, |range|)/100 wide
                    auto zero = make_constant(type, shape, 0);
                    lo = make_shared<op::v1::Minimum>(zero, input_min_range);
                    auto eps = make_shared<op::v1::Maximum>(make_constant(type, shape, 1), max_abs(input_min_range, input_max_range)) /
                               make_constant(type, shape, 100);
                    hi = make_shared<op::v1::Maximum>(input_max_range, lo + eps);
                    hi = make_shared<op::v1::Maximum>(zero, hi);
                }
                const size_t bw = quant_type.bitwidth();
                const float range = static_cast<float>((quant_type.is_signed() ? pow(2, (bw - 1)) : pow(2, bw)) - 1);
                return max_abs(lo, hi) / make_constant(type, shape, range);
            }

            shared_ptr<Node> get_bias_scale(Output<Node> min_input, Output<Node> max_input, Output<Node> min_filter, Output<Node> max_filter)
            {
                same_type_and_shape("get_bias_scale", {min_input, max_input, min_filter, max_filter});
                auto range = make_constant(min_input.get_element_type(),
                                           min_input.get_shape(),
                                           numeric_limits<uint8_t>::max() * numeric_limits<int8_t>::max());
                return (max_abs(min_input, max_input) * max_abs(min_filter, max_filter)) / range;
            }

            shared_ptr<Node> get_sum_scale(Output<Node> min_out_1, Output<Node> max_out_1, Output<Node> min_out_2, Output<Node> max_out_2)
            {
                same_type_and_shape("get_sum_scale", {min_out_1, max_out_1, min_out_2, max_out_2});
                return max_abs(min_out_2, max_out_2) / max_abs(min_out_1, max_out_1);
            }

            shared_ptr<Node> get_dot_scale(Output<Node> min_input,
                                           Output<Node> max_input,
                                           Output<Node> min_filter,
                                           Output<Node> max_filter,
                                           Output<Node> min_freezed_output,
                                           Output<Node> max_freezed_output,
                                           const element::Type& input_type,
                                           const element::Type& output_type,
                                           const bool requantize)
            {
                same_type_and_shape("get_dot_scale", {min_input, max_input, min_filter, max_filter, min_freezed_output, max_freezed_output});
                auto data_scale = get_scale(min_input, max_input, input_type);
                auto weight_scale = get_scale(min_filter, max_filter, element::i8);
                auto out_scale = get_scale(min_freezed_output, max_freezed_output, output_type);
                if (requantize)
                    return data_scale * weight_scale / out_scale;
                return data_scale * weight_scale;
            }
        }

        using namespace quantization_utils;

        shared_ptr<Node> QuantizeBuilder(const Output<Node>& input,
                                         const Output<Node>& min,
                                         const Output<Node>& max,
                                         const element::Type& quant_type,
                                         const AxisSet& axes,
                                         op::v0::Quantize::RoundMode round_mode)
        {
            const auto real_type = input.get_element_type();
            if (min.get_element_type() != real_type)
                throw ngraph_error("QuantizeBuilder: min must match input type");
            if (max.get_element_type() != real_type)
                throw ngraph_error("QuantizeBuilder: max must match input type");
            if (min.get_shape() != max.get_shape())
                throw ngraph_error("QuantizeBuilder: min and max must have same shape");
            auto zero = make_constant(quant_type, min.get_shape(), 0);
            auto scale = get_scale(min, max, quant_type, true);
            return make_shared<op::v0::Quantize>(input, scale, zero, quant_type, axes, round_mode);
        }

        shared_ptr<Node> DequantizeBuilder(const Output<Node>& input,
                                           const Output<Node>& min,
                                           const Output<Node>& max,
                                           const element::Type& real_type,
                                           const AxisSet& axes)
        {
            const auto quant_type = input.get_element_type();
            if (min.get_element_type() != real_type)
                throw ngraph_error("DequantizeBuilder: min must match input type");
            if (max.get_element_type() != real_type)
                throw ngraph_error("DequantizeBuilder: max must match input type");
            if (min.get_shape() != max.get_shape())
                throw ngraph_error("DequantizeBuilder: min and max must have same shape");
            auto zero = make_constant(quant_type, min.get_shape(), 0);
            auto scale = get_scale(min, max, quant_type);
            return make_shared<op::v0::Dequantize>(input, scale, zero, real_type, axes);
        }

        shared_ptr<Node> QuantizedConvolutionBuilder(const Output<Node>& input,
                                                     const Output<Node>& filters,
                                                     const Strides& window_movement_strides,
                                                     const Strides& window_dilation_strides,
                                                     const CoordinateDiff& padding_below,
                                                     const CoordinateDiff& padding_above,
                                                     const Strides& data_dilation_strides,
                                                     const Output<Node>& min_input,
                                                     const Output<Node>& max_input,
                                                     const Output<Node>& min_filter,
                                                     const Output<Node>& max_filter,
                                                     const Output<Node>& min_output,
                                                     const Output<Node>& max_output,
                                                     const element::Type& output_type,
                                                     const AxisSet& input_axes,
                                                     const AxisSet& filter_axes,
                                                     const AxisSet& output_axes)
        {
            auto input_scale = get_scale(min_input, max_input, input.get_element_type());
            auto filter_scale = get_scale(min_filter, max_filter, filters.get_element_type());
            auto output_scale = get_scale(min_output, max_output, output_type);
            // builders fix every zero point at 0; the output zero point is typed like the filter
            // (quantized_conv_builder.cpp:53-78), which matches the output type in the cases built
            auto input_zero_point = op::v0::Constant::create(input.get_element_type(), Shape{}, {0});
            auto filter_zero_point = op::v0::Constant::create(filters.get_element_type(), Shape{}, {0});
            return make_shared<op::v0::QuantizedConvolution>(input, filters, window_movement_strides, window_dilation_strides, padding_below,
                                                             padding_above, data_dilation_strides, input_scale, input_zero_point, filter_scale,
                                                             filter_zero_point, output_scale, filter_zero_point, output_type, input_axes,
                                                             filter_axes, output_axes);
        }

        // i32 bias as is; any other type is quantized to i32 at the bias scale with RNE
        static Output<Node> quantized_bias(const Output<Node>& bias,
                                           const Output<Node>& min_input,
                                           const Output<Node>& max_input,
                                           const Output<Node>& min_filter,
                                           const Output<Node>& max_filter)
        {
            if (bias.get_element_type() == element::i32)
                return bias;
            auto zero = make_constant(element::i32, min_input.get_shape(), 0);
            auto bias_scale = get_bias_scale(min_input, max_input, min_filter, max_filter);
            return make_shared<op::v0::Quantize>(bias, bias_scale, zero, element::i32, AxisSet{}, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
        }

        static shared_ptr<Node> requantization_scale(const Output<Node>& input,
                                                     const Output<Node>& filters,
                                                     const Output<Node>& min_input,
                                                     const Output<Node>& max_input,
                                                     const Output<Node>& min_filter,
                                                     const Output<Node>& max_filter,
                                                     const Output<Node>& min_output,
                                                     const Output<Node>& max_output,
                                                     const element::Type& output_et)
        {
            auto input_scale = get_scale(min_input, max_input, input.get_element_type());
            auto filter_scale = get_scale(min_filter, max_filter, filters.get_element_type());
            auto output_scale = get_scale(min_output, max_output, output_et);
            return input_scale * filter_scale / output_scale;
        }

        shared_ptr<Node> QuantizedConvolutionBiasBuilder(const Output<Node>& input,
                                                         const Output<Node>& filters,
                                                         const Output<Node>& bias,
                                                         const Strides& window_movement_strides,
                                                         const Strides& window_dilation_strides,
                                                         const CoordinateDiff& padding_below,
                                                         const CoordinateDiff& padding_above,
                                                         const Strides& data_dilation_strides,
                                                         const Output<Node>& min_input,
                                                         const Output<Node>& max_input,
                                                         const Output<Node>& min_filter,
                                                         const Output<Node>& max_filter,
                                                         const Output<Node>& min_output,
                                                         const Output<Node>& max_output,
                                                         const bool with_relu)
        {
            auto output_et = with_relu ? element::u8 : element::i8;
            auto scale = requantization_scale(input, filters, min_input, max_input, min_filter, max_filter, min_output, max_output, output_et);
            auto mybias = quantized_bias(bias, min_input, max_input, min_filter, max_filter);
            return make_shared<op::v0::QuantizedConvolutionBias>(input, filters, mybias, window_movement_strides, window_dilation_strides,
                                                                 padding_below, padding_above, data_dilation_strides, scale, with_relu);
        }

        shared_ptr<Node> QuantizedConvolutionReluBuilder(const Output<Node>& input,
                                                         const Output<Node>& filters,
                                                         const Strides& window_movement_strides,
                                                         const Strides& window_dilation_strides,
                                                         const CoordinateDiff& padding_below,
                                                         const CoordinateDiff& padding_above,
                                                         const Strides& data_dilation_strides,
                                                         const Output<Node>& min_input,
                                                         const Output<Node>& max_input,
                                                         const Output<Node>& min_filter,
                                                         const Output<Node>& max_filter,
                                                         const Output<Node>& min_output,
                                                         const Output<Node>& max_output)
        {
            auto scale = requantization_scale(input, filters, min_input, max_input, min_filter, max_filter, min_output, max_output, element::u8);
            return make_shared<op::v0::QuantizedConvolutionRelu>(input, filters, window_movement_strides, window_dilation_strides, padding_below,
                                                                 padding_above, data_dilation_strides, scale);
        }

        shared_ptr<Node> QuantizedConvolutionBiasAddBuilder(const Output<Node>& input,
                                                            const Output<Node>& filters,
                                                            const Output<Node>& bias,
                                                            const Output<Node>& sum_input,
                                                            const Strides& window_movement_strides,
                                                            const Strides& window_dilation_strides,
                                                            const CoordinateDiff& padding_below,
                                                            const CoordinateDiff& padding_above,
                                                            const Strides& data_dilation_strides,
                                                            const Output<Node>& min_input,
                                                            const Output<Node>& max_input,
                                                            const Output<Node>& min_filter,
                                                            const Output<Node>& max_filter,
                                                            const Output<Node>& min_output,
                                                            const Output<Node>& max_output,
                                                            const Output<Node>& min_sum_input,
                                                            const Output<Node>& max_sum_input,
                                                            const bool with_relu)
        {
            auto output_et = with_relu ? element::u8 : element::i8;
            auto scale = requantization_scale(input, filters, min_input, max_input, min_filter, max_filter, min_output, max_output, output_et);
            auto sum_scale = get_sum_scale(min_output, max_output, min_sum_input, max_sum_input);
            auto mybias = quantized_bias(bias, min_input, max_input, min_filter, max_filter);
            return make_shared<op::v0::QuantizedConvolutionBiasAdd>(input, filters, mybias, sum_input, window_movement_strides,
                                                                    window_dilation_strides, padding_below, padding_above,
                                                                    data_dilation_strides, scale, sum_scale, with_relu);
        }

        shared_ptr<Node> QuantizedConvolutionBiasSignedAddBuilder(const Output<Node>& input,
                                                                  const Output<Node>& filters,
                                                                  const Output<Node>& bias,
                                                                  const Output<Node>& sum_input,
                                                                  const Strides& window_movement_strides,
                                                                  const Strides& window_dilation_strides,
                                                                  const CoordinateDiff& padding_below,
                                                                  const CoordinateDiff& padding_above,
                                                                  const Strides& data_dilation_strides,
                                                                  const Output<Node>& min_input,
                                                                  const Output<Node>& max_input,
                                                                  const Output<Node>& min_filter,
                                                                  const Output<Node>& max_filter,
                                                                  const Output<Node>& min_output,
                                                                  const Output<Node>& max_output,
                                                                  const Output<Node>& min_sum_input,
                                                                  const Output<Node>& max_sum_input,
                                                                  const bool with_relu)
        {
            auto output_et = with_relu ? element::u8 : element::i8;
            auto scale = requantization_scale(input, filters, min_input, max_input, min_filter, max_filter, min_output, max_output, output_et);
            shared_ptr<Node> sum_scale = get_sum_scale(min_output, max_output, min_sum_input, max_sum_input);
            if (output_et == element::u8)
            {
                // the requantization scale targets u8 (255 steps) while the sum input is i8 (127):
                // doubling the sum scale puts both on the same grid
                sum_scale = make_constant(element::f32, sum_scale->get_output_shape(0), 2.0f) * sum_scale;
            }
            auto mybias = quantized_bias(bias, min_input, max_input, min_filter, max_filter);
            auto qconv = make_shared<op::v0::QuantizedConvolutionBiasSignedAdd>(input, filters, mybias, sum_input, window_movement_strides,
                                                                                window_dilation_strides, padding_below, padding_above,
                                                                                data_dilation_strides, scale, sum_scale, with_relu);
            return make_shared<op::v0::Convert>(qconv, element::u8);
        }

        shared_ptr<Node> QuantizedDotBuilder(const Output<Node>& input0,
                                             const Output<Node>& input1,
                                             const size_t reduction_axes_count,
                                             const Output<Node>& min_input0,
                                             const Output<Node>& max_input0,
                                             const Output<Node>& min_input1,
                                             const Output<Node>& max_input1,
                                             const Output<Node>& min_output,
                                             const Output<Node>& max_output,
                                             const element::Type& output_type,
                                             const AxisSet& input0_axes,
                                             const AxisSet& input1_axes,
                                             const AxisSet& output_axes)
        {
            auto input0_scale = get_scale(min_input0, max_input0, input0.get_element_type());
            auto input1_scale = get_scale(min_input1, max_input1, input1.get_element_type());
            auto output_scale = get_scale(min_output, max_output, output_type);
            auto input0_zero_point = op::v0::Constant::create(input0.get_element_type(), Shape{}, {0});
            auto input1_zero_point = op::v0::Constant::create(input1.get_element_type(), Shape{}, {0});
            auto output_zero_point = op::v0::Constant::create(output_type, Shape{}, {0});
            return make_shared<op::v0::QuantizedDot>(input0, input1, reduction_axes_count, input0_scale, input0_zero_point, input1_scale,
                                                     input1_zero_point, output_scale, output_zero_point, output_type, input0_axes, input1_axes,
                                                     output_axes);
        }

        shared_ptr<Node> QuantizedDotBiasBuilder(const Output<Node>& input,
                                                 const Output<Node>& filters,
                                                 const Output<Node>& bias,
                                                 const Output<Node>& min_input,
                                                 const Output<Node>& max_input,
                                                 const Output<Node>& min_filter,
                                                 const Output<Node>& max_filter,
                                                 const Output<Node>& min_output,
                                                 const Output<Node>& max_output,
                                                 const bool requantize,
                                                 const bool with_relu)
        {
            auto scale = get_dot_scale(min_input, max_input, min_filter, max_filter, min_output, max_output, input.get_element_type(),
                                       with_relu ? element::u8 : element::i8, requantize);
            auto mybias = quantized_bias(bias, min_input, max_input, min_filter, max_filter);
            return make_shared<op::v0::QuantizedDotBias>(input, filters, mybias, scale, requantize, with_relu);
        }
    }
}
