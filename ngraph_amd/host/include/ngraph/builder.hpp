// Graph builders of the quantized ops: they take (min, max) ranges and emit the f32 sub-graph that
// derives scales, with zero points fixed at 0.
//
// Mirrors src/ngraph/builder/{make_constant.hpp, quantization_utils.{hpp,cpp}, quantize_builder,
// dequantize_builder, quantized_conv_builder, quantized_dot_builder}.{hpp,cpp} of the nGraph tree.
#pragma once

#include "ngraph/ops.hpp"

namespace ngraph
{
    namespace builder
    {
        // constant of `shape` filled with `num` (the reference emits scalar Constant + Broadcast)
        template <typename T>
        std::shared_ptr<Node> make_constant(const element::Type& type, const Shape& shape, const T& num)
        {
            return op::v0::Constant::create(type, shape, std::vector<T>{num});
        }

        namespace quantization_utils
        {
            NGRAPH_API std::shared_ptr<Node> max_abs(const Output<Node>& a, const Output<Node>& b);
            // scale = max(|min|, |max|) / (2^(bw-1)-1 signed, 2^bw-1 unsigned); bump_by_eps widens
            // the range the way QuantizeBuilder wants (quantization_utils.cpp:33-79)
            NGRAPH_API std::shared_ptr<Node> get_scale(const Output<Node>& input_min_range,
                                                       const Output<Node>& input_max_range,
                                                       const element::Type& quant_type,
                                                       bool bump_by_eps = false);
            NGRAPH_API std::shared_ptr<Node> get_bias_scale(Output<Node> min_input,
                                                            Output<Node> max_input,
                                                            Output<Node> min_filter,
                                                            Output<Node> max_filter);
            NGRAPH_API std::shared_ptr<Node> get_sum_scale(Output<Node> min_freezed_output_conv_1,
                                                           Output<Node> max_freezed_output_conv_1,
                                                           Output<Node> min_freezed_output_conv_2,
                                                           Output<Node> max_freezed_output_conv_2);
            NGRAPH_API std::shared_ptr<Node> get_dot_scale(Output<Node> min_input,
                                                           Output<Node> max_input,
                                                           Output<Node> min_filter,
                                                           Output<Node> max_filter,
                                                           Output<Node> min_freezed_output,
                                                           Output<Node> max_freezed_output,
                                                           const element::Type& input_type,
                                                           const element::Type& output_type,
                                                           const bool requantize = true);
        }

        NGRAPH_API std::shared_ptr<Node> QuantizeBuilder(const Output<Node>& input,
                                                         const Output<Node>& min,
                                                         const Output<Node>& max,
                                                         const element::Type& quant_type,
                                                         const AxisSet& axes,
                                                         op::v0::Quantize::RoundMode round_mode);

        NGRAPH_API std::shared_ptr<Node> DequantizeBuilder(const Output<Node>& input,
                                                           const Output<Node>& min,
                                                           const Output<Node>& max,
                                                           const element::Type& real_type,
                                                           const AxisSet& axes);

        NGRAPH_API std::shared_ptr<Node> QuantizedConvolutionBuilder(const Output<Node>& input,
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
                                                                     const AxisSet& input_axes = AxisSet{},
                                                                     const AxisSet& filter_axes = AxisSet{},
                                                                     const AxisSet& output_axes = AxisSet{});

        NGRAPH_API std::shared_ptr<Node> QuantizedConvolutionBiasBuilder(const Output<Node>& input,
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
                                                                         const bool with_relu = false);

        NGRAPH_API std::shared_ptr<Node> QuantizedConvolutionReluBuilder(const Output<Node>& input,
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
                                                                         const Output<Node>& max_output);

        NGRAPH_API std::shared_ptr<Node> QuantizedConvolutionBiasAddBuilder(const Output<Node>& input,
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
                                                                            const bool with_relu = false);

        NGRAPH_API std::shared_ptr<Node> QuantizedConvolutionBiasSignedAddBuilder(const Output<Node>& input,
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
                                                                                  const bool with_relu = false);

        NGRAPH_API std::shared_ptr<Node> QuantizedDotBuilder(const Output<Node>& input0,
                                                             const Output<Node>& input1,
                                                             const size_t reduction_axes_count,
                                                             const Output<Node>& min_input0,
                                                             const Output<Node>& max_input0,
                                                             const Output<Node>& min_input1,
                                                             const Output<Node>& max_input1,
                                                             const Output<Node>& min_output,
                                                             const Output<Node>& max_output,
                                                             const element::Type& output_type,
                                                             const AxisSet& input0_axes = AxisSet{},
                                                             const AxisSet& input1_axes = AxisSet{},
                                                             const AxisSet& output_axes = AxisSet{});

        NGRAPH_API std::shared_ptr<Node> QuantizedDotBiasBuilder(const Output<Node>& input,
                                                                 const Output<Node>& filters,
                                                                 const Output<Node>& bias,
                                                                 const Output<Node>& min_input,
                                                                 const Output<Node>& max_input,
                                                                 const Output<Node>& min_filter,
                                                                 const Output<Node>& max_filter,
                                                                 const Output<Node>& min_output,
                                                                 const Output<Node>& max_output,
                                                                 const bool requantize = true,
                                                                 const bool with_relu = false);
    }
}
