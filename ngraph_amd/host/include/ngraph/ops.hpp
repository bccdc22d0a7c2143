// Operators of the int8 path and of the small f32 sub-graphs that derive its scales.
//
// Constructor signatures, input order, output types and validation rules follow the nGraph tree:
//   src/ngraph/op/quantize.{hpp,cpp}, dequantize.{hpp,cpp}, quantized_convolution.{hpp,cpp},
//   quantized_dot.{hpp,cpp}, src/ngraph/op/experimental/quantized_conv_bias.{hpp,cpp},
//   quantized_conv_relu.{hpp,cpp}, quantized_dot_bias.{hpp,cpp}, and for the glue ops
//   src/ngraph/op/{parameter,constant,result,abs,broadcast,convert,relu,add,multiply,divide,
//   maximum,minimum,max_pool,avg_pool}.hpp.
#pragma once

#include <cstring>
#include <initializer_list>

#include "ngraph/core.hpp"

#define NGRAPH_OP_DECL(NAME, VERSION)                                                              \
    static constexpr NodeTypeInfo type_info{NAME, VERSION};                                        \
    const NodeTypeInfo& get_type_info() const override { return type_info; }

namespace ngraph
{
    namespace op
    {
        namespace v0
        {
            class NGRAPH_API Parameter : public Op
            {
            public:
                NGRAPH_OP_DECL("Parameter", 0)
                Parameter(const element::Type& type, const Shape& shape);
                bool is_parameter() const override { return true; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;
            };

            class NGRAPH_API Result : public Op
            {
            public:
                NGRAPH_OP_DECL("Result", 0)
                explicit Result(const Output<Node>& arg);
                bool is_output() const override { return true; }
                void validate_and_infer_types() override;
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;
            };

            class NGRAPH_API Constant : public Op
            {
            public:
                NGRAPH_OP_DECL("Constant", 0)
                Constant(const element::Type& type, const Shape& shape, const void* data);
                template <typename T>
                Constant(const element::Type& type, const Shape& shape, const std::vector<T>& values)
                {
                    init(type, shape);
                    NGRAPH_CHECK(values.size() == 1 || values.size() == shape_size(shape),
                                 "Did not get the expected number of literals for a constant of shape ",
                                 shape,
                                 " (got ",
                                 values.size(),
                                 ")");
                    std::vector<double> v(values.begin(), values.end());
                    fill(v);
                }
                template <typename T>
                static std::shared_ptr<Constant> create(const element::Type& type, const Shape& shape, const std::vector<T>& values)
                {
                    return std::make_shared<Constant>(type, shape, values);
                }
                template <typename T>
                static std::shared_ptr<Constant> create(const element::Type& type, const Shape& shape, std::initializer_list<T> values)
                {
                    return std::make_shared<Constant>(type, shape, std::vector<T>(values));
                }
                bool is_constant() const override { return true; }
                const void* get_data_ptr() const { return m_data.data(); }
                template <typename T>
                const T* get_data_ptr() const
                {
                    return reinterpret_cast<const T*>(m_data.data());
                }
                template <typename T>
                std::vector<T> get_vector() const
                {
                    NGRAPH_CHECK(element::from<T>() == get_output_element_type(0) || sizeof(T) == get_output_element_type(0).size(),
                                 "get_vector type does not match the constant's element type");
                    const T* p = get_data_ptr<T>();
                    return std::vector<T>(p, p + shape_size(get_output_shape(0)));
                }
                // values converted to double, whatever the element type
                std::vector<double> get_values_as_double() const;
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                void init(const element::Type& type, const Shape& shape);
                void fill(const std::vector<double>& values);
                std::vector<uint8_t> m_data;
            };

            // ---- unary / shape glue --------------------------------------------------------------
            class NGRAPH_API Abs : public Op
            {
            public:
                NGRAPH_OP_DECL("Abs", 0)
                explicit Abs(const Output<Node>& arg);
                void validate_and_infer_types() override;
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;
            };

            class NGRAPH_API Relu : public Op
            {
            public:
                NGRAPH_OP_DECL("Relu", 0)
                explicit Relu(const Output<Node>& arg);
                void validate_and_infer_types() override;
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;
            };

            class NGRAPH_API Convert : public Op
            {
            public:
                NGRAPH_OP_DECL("Convert", 0)
                Convert(const Output<Node>& arg, const element::Type& destination_type);
                void validate_and_infer_types() override;
                const element::Type& get_destination_type() const { return m_type; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                element::Type m_type;
            };

            class NGRAPH_API Broadcast : public Op
            {
            public:
                NGRAPH_OP_DECL("Broadcast", 0)
                Broadcast(const Output<Node>& arg, const Shape& shape, const AxisSet& broadcast_axes);
                void validate_and_infer_types() override;
                const Shape& get_broadcast_shape() const { return m_shape; }
                const AxisSet& get_broadcast_axes() const { return m_axes; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                Shape m_shape;
                AxisSet m_axes;
            };

            // Reshape with an input axis order: a transpose followed by a reinterpretation
            class NGRAPH_API Reshape : public Op
            {
            public:
                NGRAPH_OP_DECL("Reshape", 0)
                Reshape(const Output<Node>& arg, const AxisVector& input_order, const Shape& output_shape);
                void validate_and_infer_types() override;
                const AxisVector& get_input_order() const { return m_order; }
                const Shape& get_reshape_output_shape() const { return m_shape; }
                bool get_is_transpose() const;
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                AxisVector m_order;
                Shape m_shape;
            };

            // ---- Quantize / Dequantize -------------------------------------------------------------
            class NGRAPH_API Quantize : public Op
            {
            public:
                NGRAPH_OP_DECL("Quantize", 0)
                enum class RoundMode
                {
                    ROUND_NEAREST_TOWARD_INFINITY,
                    ROUND_NEAREST_TOWARD_ZERO,
                    ROUND_NEAREST_UPWARD,
                    ROUND_NEAREST_DOWNWARD,
                    ROUND_NEAREST_TOWARD_EVEN,
                    ROUND_TOWARD_INFINITY,
                    ROUND_TOWARD_ZERO,
                    ROUND_UP,
                    ROUND_DOWN
                };
                Quantize(const Output<Node>& input,
                         const Output<Node>& scale,
                         const Output<Node>& zero_point,
                         const element::Type& type,
                         const AxisSet& axes,
                         RoundMode round_mode);
                void validate_and_infer_types() override;
                const AxisSet& get_axes() const { return m_axes; }
                RoundMode get_round_mode() const { return m_round_mode; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                element::Type m_type;
                AxisSet m_axes;
                RoundMode m_round_mode;
            };

            class NGRAPH_API Dequantize : public Op
            {
            public:
                NGRAPH_OP_DECL("Dequantize", 0)
                Dequantize(const Output<Node>& input,
                           const Output<Node>& scale,
                           const Output<Node>& zero_point,
                           const element::Type& type,
                           const AxisSet& axes);
                void validate_and_infer_types() override;
                const AxisSet& get_axes() const { return m_axes; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                element::Type m_type;
                AxisSet m_axes;
            };

            // ---- convolutions ------------------------------------------------------------------------
            // attributes shared by the five quantized convolution ops
            class NGRAPH_API ConvAttributes
            {
            public:
                const Strides& get_window_movement_strides() const { return m_window_movement_strides; }
                const Strides& get_window_dilation_strides() const { return m_window_dilation_strides; }
                const CoordinateDiff& get_padding_below() const { return m_padding_below; }
                const CoordinateDiff& get_padding_above() const { return m_padding_above; }
                const Strides& get_data_dilation_strides() const { return m_data_dilation_strides; }

            protected:
                ConvAttributes() = default;
                ConvAttributes(const Strides& s, const Strides& d, const CoordinateDiff& pb, const CoordinateDiff& pa, const Strides& dd)
                    : m_window_movement_strides(s), m_window_dilation_strides(d), m_padding_below(pb), m_padding_above(pa), m_data_dilation_strides(dd)
                {
                }
                Strides m_window_movement_strides;
                Strides m_window_dilation_strides;
                CoordinateDiff m_padding_below;
                CoordinateDiff m_padding_above;
                Strides m_data_dilation_strides;
            };

            class NGRAPH_API QuantizedConvolution : public Op, public ConvAttributes
            {
            public:
                NGRAPH_OP_DECL("QuantizedConvolution", 0)
                QuantizedConvolution(const Output<Node>& input,
                                     const Output<Node>& filters,
                                     const Strides& window_movement_strides,
                                     const Strides& window_dilation_strides,
                                     const CoordinateDiff& padding_below,
                                     const CoordinateDiff& padding_above,
                                     const Strides& data_dilation_strides,
                                     const Output<Node>& input_scale,
                                     const Output<Node>& input_zero_point,
                                     const Output<Node>& filter_scale,
                                     const Output<Node>& filter_zero_point,
                                     const Output<Node>& output_scale,
                                     const Output<Node>& output_zero_point,
                                     const element::Type& output_type,
                                     const AxisSet& input_axes = AxisSet{},
                                     const AxisSet& filter_axes = AxisSet{},
                                     const AxisSet& output_axes = AxisSet{});
                void validate_and_infer_types() override;
                const element::Type& get_output_type() const { return m_output_type; }
                const AxisSet& get_input_axes() const { return m_input_axes; }
                const AxisSet& get_filter_axes() const { return m_filter_axes; }
                const AxisSet& get_output_axes() const { return m_output_axes; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                element::Type m_output_type;
                AxisSet m_input_axes, m_filter_axes, m_output_axes;
            };

            // inputs {data, filters, bias, scale}; output i8, or u8 with relu
            class NGRAPH_API QuantizedConvolutionBias : public Op, public ConvAttributes
            {
            public:
                NGRAPH_OP_DECL("QuantizedConvolutionBias", 0)
                QuantizedConvolutionBias(const Output<Node>& data_batch,
                                         const Output<Node>& filters,
                                         const Output<Node>& bias,
                                         const Strides& window_movement_strides,
                                         const Strides& window_dilation_strides,
                                         const CoordinateDiff& padding_below,
                                         const CoordinateDiff& padding_above,
                                         const Strides& data_dilation_strides,
                                         const Output<Node>& scale,
                                         const bool with_relu = false);
                bool with_relu() const { return m_with_relu; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                bool m_with_relu;
            };

            // inputs {data, filters, scale}; always relu, output u8
            class NGRAPH_API QuantizedConvolutionRelu : public Op, public ConvAttributes
            {
            public:
                NGRAPH_OP_DECL("QuantizedConvolutionRelu", 0)
                QuantizedConvolutionRelu(const Output<Node>& data_batch,
                                         const Output<Node>& filters,
                                         const Strides& window_movement_strides,
                                         const Strides& window_dilation_strides,
                                         const CoordinateDiff& padding_below,
                                         const CoordinateDiff& padding_above,
                                         const Strides& data_dilation_strides,
                                         const Output<Node>& scale);
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;
            };

            // inputs {data, filters, bias, sum_input, scale, sum_scale}; output i8, or u8 with relu
            class NGRAPH_API QuantizedConvolutionBiasAdd : public Op, public ConvAttributes
            {
            public:
                NGRAPH_OP_DECL("QuantizedConvolutionBiasAdd", 0)
                QuantizedConvolutionBiasAdd(const Output<Node>& data_batch,
                                            const Output<Node>& filters,
                                            const Output<Node>& bias,
                                            const Output<Node>& sum_input,
                                            const Strides& window_movement_strides,
                                            const Strides& window_dilation_strides,
                                            const CoordinateDiff& padding_below,
                                            const CoordinateDiff& padding_above,
                                            const Strides& data_dilation_strides,
                                            const Output<Node>& scale,
                                            const Output<Node>& sum_scale,
                                            const bool with_relu = false);
                bool with_relu() const { return m_with_relu; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                bool m_with_relu;
            };

            // as BiasAdd with an i8 sum input; output stays i8 even with relu
            class NGRAPH_API QuantizedConvolutionBiasSignedAdd : public Op, public ConvAttributes
            {
            public:
                NGRAPH_OP_DECL("QuantizedConvolutionBiasSignedAdd", 0)
                QuantizedConvolutionBiasSignedAdd(const Output<Node>& data_batch,
                                                  const Output<Node>& filters,
                                                  const Output<Node>& bias,
                                                  const Output<Node>& sum_input,
                                                  const Strides& window_movement_strides,
                                                  const Strides& window_dilation_strides,
                                                  const CoordinateDiff& padding_below,
                                                  const CoordinateDiff& padding_above,
                                                  const Strides& data_dilation_strides,
                                                  const Output<Node>& scale,
                                                  const Output<Node>& sum_scale,
                                                  const bool with_relu = false);
                bool with_relu() const { return m_with_relu; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                bool m_with_relu;
            };

            // ---- dots ----------------------------------------------------------------------------------
            class NGRAPH_API QuantizedDot : public Op
            {
            public:
                NGRAPH_OP_DECL("QuantizedDot", 0)
                QuantizedDot(const Output<Node>& input0,
                             const Output<Node>& input1,
                             size_t reduction_axes_count,
                             const Output<Node>& input0_scale,
                             const Output<Node>& input0_zero_point,
                             const Output<Node>& input1_scale,
                             const Output<Node>& input1_zero_point,
                             const Output<Node>& output_scale,
                             const Output<Node>& output_zero_point,
                             const element::Type& output_type,
                             const AxisSet& input0_axes = AxisSet{},
                             const AxisSet& input1_axes = AxisSet{},
                             const AxisSet& output_axes = AxisSet{});
                void validate_and_infer_types() override;
                size_t get_reduction_axes_count() const { return m_reduction_axes_count; }
                const element::Type& get_output_type() const { return m_output_type; }
                const AxisSet& get_input0_axes() const { return m_input0_axes; }
                const AxisSet& get_input1_axes() const { return m_input1_axes; }
                const AxisSet& get_output_axes() const { return m_output_axes; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                size_t m_reduction_axes_count;
                element::Type m_output_type;
                AxisSet m_input0_axes, m_input1_axes, m_output_axes;
            };

            // inputs {data [M,K], weights [N,K], bias [N], scale}
            class NGRAPH_API QuantizedDotBias : public Op
            {
            public:
                NGRAPH_OP_DECL("QuantizedDotBias", 0)
                QuantizedDotBias(const Output<Node>& data,
                                 const Output<Node>& weights,
                                 const Output<Node>& bias,
                                 const Output<Node>& scale,
                                 bool requantize = true,
                                 bool with_relu = false);
                bool with_relu() const { return m_with_relu; }
                bool requantize() const { return m_requantize; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                bool m_requantize;
                bool m_with_relu;
            };

            // ---- pooling (integer glue of quantized networks) --------------------------------------------
            class NGRAPH_API MaxPool : public Op
            {
            public:
                NGRAPH_OP_DECL("MaxPool", 0)
                MaxPool(const Output<Node>& arg,
                        const Shape& window_shape,
                        const Strides& window_movement_strides,
                        const Shape& padding_below,
                        const Shape& padding_above);
                void validate_and_infer_types() override;
                const Shape& get_window_shape() const { return m_window_shape; }
                const Strides& get_window_movement_strides() const { return m_strides; }
                const Shape& get_padding_below() const { return m_padding_below; }
                const Shape& get_padding_above() const { return m_padding_above; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                Shape m_window_shape;
                Strides m_strides;
                Shape m_padding_below, m_padding_above;
            };

            class NGRAPH_API AvgPool : public Op
            {
            public:
                NGRAPH_OP_DECL("AvgPool", 0)
                AvgPool(const Output<Node>& arg,
                        const Shape& window_shape,
                        const Strides& window_movement_strides,
                        const Shape& padding_below,
                        const Shape& padding_above,
                        bool include_padding_in_avg_computation = false);
                void validate_and_infer_types() override;
                const Shape& get_window_shape() const { return m_window_shape; }
                const Strides& get_window_movement_strides() const { return m_strides; }
                const Shape& get_padding_below() const { return m_padding_below; }
                const Shape& get_padding_above() const { return m_padding_above; }
                bool get_include_padding_in_avg_computation() const { return m_include_padding; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                Shape m_window_shape;
                Strides m_strides;
                Shape m_padding_below, m_padding_above;
                bool m_include_padding;
            };

            // joins tensors that agree on every axis but `axis` (src/ngraph/op/concat.hpp:30-68);
            // a negative axis counts from the back
            class NGRAPH_API Concat : public Op
            {
            public:
                NGRAPH_OP_DECL("Concat", 0)
                Concat(const OutputVector& args, int64_t axis);
                void validate_and_infer_types() override;
                int64_t get_concatenation_axis() const { return m_concat_axis; }
                int64_t get_axis() const { return m_axis; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                int64_t m_axis;
                int64_t m_concat_axis = -1;
            };

            // src/ngraph/op/slice.hpp:28-76: the elements lower_bounds + i * strides < upper_bounds of every axis
            class NGRAPH_API Slice : public Op
            {
            public:
                NGRAPH_OP_DECL("Slice", 0)
                Slice(const Output<Node>& arg, const Coordinate& lower_bounds, const Coordinate& upper_bounds, const Strides& strides);
                Slice(const Output<Node>& arg, const Coordinate& lower_bounds, const Coordinate& upper_bounds);
                void validate_and_infer_types() override;
                const Coordinate& get_lower_bounds() const { return m_lower_bounds; }
                const Coordinate& get_upper_bounds() const { return m_upper_bounds; }
                const Strides& get_strides() const { return m_strides; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                Coordinate m_lower_bounds, m_upper_bounds;
                Strides m_strides;
            };

            // ---- fp32 glue of a transformer encoder --------------------------------------------------
            // src/ngraph/op/softmax.hpp:28-60 (static axes)
            class NGRAPH_API Softmax : public Op
            {
            public:
                NGRAPH_OP_DECL("Softmax", 0)
                Softmax(const Output<Node>& arg, const AxisSet& axes);
                void validate_and_infer_types() override;
                const AxisSet& get_axes() const { return m_axes; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;

            private:
                AxisSet m_axes;
            };

            // src/ngraph/op/erf.hpp
            class NGRAPH_API Erf : public Op
            {
            public:
                NGRAPH_OP_DECL("Erf", 0)
                explicit Erf(const Output<Node>& arg);
                void validate_and_infer_types() override;
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;
            };

            // src/ngraph/op/gelu.hpp:30-50: 0.5 * x * (1 + erf(x / sqrt(2)))
            class NGRAPH_API Gelu : public Op
            {
            public:
                NGRAPH_OP_DECL("Gelu", 0)
                explicit Gelu(const Output<Node>& arg);
                void validate_and_infer_types() override;
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;
            };

            // src/ngraph/op/layer_norm.hpp:31-80 (forward): outputs norm, and mean and variance
            // over the normalised axes when keep_stats
            class NGRAPH_API LayerNorm : public Op
            {
            public:
                NGRAPH_OP_DECL("LayerNorm", 0)
                LayerNorm(const Output<Node>& data, const Output<Node>& scale, const Output<Node>& bias, bool keep_stats = true, int64_t begin_norm_axis = 1, double epsilon = 1e-5);
                LayerNorm(const Output<Node>& data, bool keep_stats = true, int64_t begin_norm_axis = 1, double epsilon = 1e-5);
                void validate_and_infer_types() override;
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;
                bool get_keep_stats() const { return m_keep_stats; }
                bool get_use_affine() const { return m_use_affine; }
                double get_epsilon() const { return m_epsilon; }
                int64_t get_begin_norm_axis() const { return m_begin_norm_axis; }

            private:
                bool m_keep_stats{true};
                bool m_use_affine{true};
                int64_t m_begin_norm_axis{1};
                double m_epsilon{1e-5};
            };

            // src/ngraph/op/experimental/batch_mat_mul.hpp: [b, m, k] x [b, k, n] -> [b, m, n]
            class NGRAPH_API BatchMatMul : public Op
            {
            public:
                NGRAPH_OP_DECL("BatchMatMul", 0)
                BatchMatMul(const Output<Node>& arg0, const Output<Node>& arg1);
                void validate_and_infer_types() override;
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;
            };

            // src/ngraph/op/batch_mat_mul_transpose.hpp: the same with either operand read transposed
            class NGRAPH_API BatchMatMulTranspose : public Op
            {
            public:
                NGRAPH_OP_DECL("BatchMatMulTranspose", 0)
                BatchMatMulTranspose(const Output<Node>& arg0, const Output<Node>& arg1, bool transpose_arg0 = false, bool transpose_arg1 = false);
                void validate_and_infer_types() override;
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override;
                bool get_transpose_arg0() const { return m_transpose_arg0; }
                bool get_transpose_arg1() const { return m_transpose_arg1; }

            private:
                bool m_transpose_arg0;
                bool m_transpose_arg1;
            };
        }

        namespace v1
        {
            // Binary elementwise with numpy broadcasting restricted to "same shape or one side has
            // a single element" (all the scale sub-graphs need).
            class NGRAPH_API BinaryElementwise : public Op
            {
            public:
                void validate_and_infer_types() override;

            protected:
                BinaryElementwise(const Output<Node>& a, const Output<Node>& b) : Op({a, b}) {}
            };

#define NGRAPH_BINARY_OP(NAME)                                                                     \
    class NGRAPH_API NAME : public BinaryElementwise                                               \
    {                                                                                              \
    public:                                                                                        \
        NGRAPH_OP_DECL(#NAME, 1)                                                                   \
        NAME(const Output<Node>& a, const Output<Node>& b) : BinaryElementwise(a, b)               \
        {                                                                                          \
            constructor_validate_and_infer_types();                                                \
        }                                                                                          \
        std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override   \
        {                                                                                          \
            check_new_args_count(this, new_args);                                                  \
            return std::make_shared<NAME>(new_args.at(0), new_args.at(1));                         \
        }                                                                                          \
    };
            NGRAPH_BINARY_OP(Add)
            NGRAPH_BINARY_OP(Subtract)
            NGRAPH_BINARY_OP(Multiply)
            // Divide carries the reference's flag (src/ngraph/op/divide.hpp:35-76): integer division
            // floors by default ("python division"), truncates with the flag off
            class NGRAPH_API Divide : public BinaryElementwise
            {
            public:
                NGRAPH_OP_DECL("Divide", 1)
                Divide(const Output<Node>& a, const Output<Node>& b, bool pythondiv = true) : BinaryElementwise(a, b), m_pythondiv(pythondiv)
                {
                    constructor_validate_and_infer_types();
                }
                bool is_pythondiv() const { return m_pythondiv; }
                void set_is_pythondiv(bool pythondiv) { m_pythondiv = pythondiv; }
                std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const override
                {
                    check_new_args_count(this, new_args);
                    return std::make_shared<Divide>(new_args.at(0), new_args.at(1), m_pythondiv);
                }

            protected:
                bool m_pythondiv{true};
            };
            NGRAPH_BINARY_OP(Maximum)
            NGRAPH_BINARY_OP(Minimum)
#undef NGRAPH_BINARY_OP
        }

        // the opset-0 names the tests use without a version
        using v0::Abs;
        using v0::AvgPool;
        using v0::BatchMatMul;
        using v0::BatchMatMulTranspose;
        using v0::Broadcast;
        using v0::Concat;
        using v0::Constant;
        using v0::Convert;
        using v0::Dequantize;
        using v0::Erf;
        using v0::Gelu;
        using v0::LayerNorm;
        using v0::MaxPool;
        using v0::Parameter;
        using v0::Quantize;
        using v0::QuantizedConvolution;
        using v0::QuantizedConvolutionBias;
        using v0::QuantizedConvolutionBiasAdd;
        using v0::QuantizedConvolutionBiasSignedAdd;
        using v0::QuantizedConvolutionRelu;
        using v0::QuantizedDot;
        using v0::QuantizedDotBias;
        using v0::Relu;
        using v0::Reshape;
        using v0::Result;
        using v0::Slice;
        using v0::Softmax;
    }

    NGRAPH_API std::shared_ptr<Node> operator+(const Output<Node>& a, const Output<Node>& b);
    NGRAPH_API std::shared_ptr<Node> operator-(const Output<Node>& a, const Output<Node>& b);
    NGRAPH_API std::shared_ptr<Node> operator*(const Output<Node>& a, const Output<Node>& b);
    NGRAPH_API std::shared_ptr<Node> operator/(const Output<Node>& a, const Output<Node>& b);

    // inferred output shape of a convolution (src/ngraph/validation_util.cpp
    // infer_convolution_forward); throws NodeValidationFailure on inconsistent attributes
    NGRAPH_API Shape infer_convolution_forward(const Node* node,
                                               const Shape& data_shape,
                                               const Strides& data_dilation,
                                               const CoordinateDiff& padding_below,
                                               const CoordinateDiff& padding_above,
                                               const Shape& filters_shape,
                                               const Strides& strides,
                                               const Strides& filter_dilation);
}
