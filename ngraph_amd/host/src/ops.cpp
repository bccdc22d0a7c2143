// Operator constructors, validation and shape / type inference.
// Validation messages and rules follow src/ngraph/op/quantize.cpp:40-154, dequantize.cpp:40-140,
// quantized_convolution.cpp:64-172, quantized_dot.cpp:58-201 and the experimental fused ops of the
// nGraph tree; test/type_prop/{quantize,dequantize,quantized_convolution,quantized_dot}.cpp is the
// specification they are checked against.
#include <algorithm>
#include <cmath>
#include <limits>

#include "ngraph/ops.hpp"

using namespace std;

namespace ngraph
{
    Shape infer_convolution_forward(const Node* node,
                                    const Shape& data_shape,
                                    const Strides& data_dilation,
                                    const CoordinateDiff& padding_below,
                                    const CoordinateDiff& padding_above,
                                    const Shape& filters_shape,
                                    const Strides& strides,
                                    const Strides& filter_dilation)
    {
        NODE_VALIDATION_CHECK(node, data_shape.size() >= 3, "Data batch must have rank of at least 3 (one batch axis, one input-channel axis, and at least one spatial dimension) (data batch shape: ", data_shape, ").");
        NODE_VALIDATION_CHECK(node, filters_shape.size() == data_shape.size(), "Data batch and filters rank do not match (data batch shape: ", data_shape, ", filters shape: ", filters_shape, ").");
        const size_t ns = data_shape.size() - 2;
        NODE_VALIDATION_CHECK(node,
                              data_dilation.size() == ns && padding_below.size() == ns && padding_above.size() == ns &&
                                  strides.size() == ns && filter_dilation.size() == ns,
                              "Ranks for data item shape/filters shape (data batch has shape ",
                              data_shape,
                              ", so data item rank is ",
                              ns,
                              "), data dilation, padding below, padding above, filter strides, and filter dilation do not match.");
        NODE_VALIDATION_CHECK(node, data_shape[0] > 0, "Batch size is zero.");
        NODE_VALIDATION_CHECK(node, data_shape[1] > 0, "Data batch channel count is zero.");
        NODE_VALIDATION_CHECK(node, filters_shape[0] > 0, "Filter output channel count is zero.");
        NODE_VALIDATION_CHECK(node,
                              data_shape[1] == filters_shape[1],
                              "Data batch channel count (",
                              data_shape[1],
                              ") does not match filter input channel count (",
                              filters_shape[1],
                              ").");
        Shape out{data_shape[0], filters_shape[0]};
        for (size_t i = 0; i < ns; ++i)
        {
            NODE_VALIDATION_CHECK(node, data_dilation[i] > 0, "Data dilation (", data_dilation[i], ") has zero dimension at axis ", i, ".");
            NODE_VALIDATION_CHECK(node, strides[i] > 0, "Window strides (", strides[i], ") has zero dimension at axis ", i, ".");
            NODE_VALIDATION_CHECK(node, filter_dilation[i] > 0, "Window dilation (", filter_dilation[i], ") has zero dimension at axis ", i, ".");
            NODE_VALIDATION_CHECK(node, filters_shape[2 + i] > 0, "Window after dilation has dimension less than 1 at axis ", i, ".");
            ptrdiff_t data_eff = (static_cast<ptrdiff_t>(data_shape[2 + i]) - 1) * static_cast<ptrdiff_t>(data_dilation[i]) + 1 +
                                 padding_below[i] + padding_above[i];
            ptrdiff_t win_eff = (static_cast<ptrdiff_t>(filters_shape[2 + i]) - 1) * static_cast<ptrdiff_t>(filter_dilation[i]) + 1;
            NODE_VALIDATION_CHECK(node, data_eff > 0, "Data shape after padding and dilation has dimension less than 1 (dim: ", data_eff, ") at axis ", i, ".");
            NODE_VALIDATION_CHECK(node,
                                  win_eff <= data_eff,
                                  "Window after dilation has dimension (dim: ",
                                  win_eff,
                                  ") larger than the data shape after padding (dim: ",
                                  data_eff,
                                  ") at axis ",
                                  i,
                                  ".");
            out.push_back(static_cast<size_t>((data_eff - win_eff) / static_cast<ptrdiff_t>(strides[i]) + 1));
        }
        return out;
    }

    namespace op
    {
        namespace v0
        {
            constexpr NodeTypeInfo Parameter::type_info;
            constexpr NodeTypeInfo Result::type_info;
            constexpr NodeTypeInfo Constant::type_info;

            // ---------------------------------------------------------------- Parameter / Result
            Parameter::Parameter(const element::Type& type, const Shape& shape) { set_output_type(0, type, shape); }
            shared_ptr<Node> Parameter::clone_with_new_inputs(const OutputVector& new_args) const
            {
                check_new_args_count(this, new_args);
                return make_shared<Parameter>(get_output_element_type(0), get_output_shape(0));
            }

            Result::Result(const Output<Node>& arg) : Op({arg}) { constructor_validate_and_infer_types(); }
            void Result::validate_and_infer_types() { set_output_type(0, get_input_element_type(0), get_input_shape(0)); }
            shared_ptr<Node> Result::clone_with_new_inputs(const OutputVector& new_args) const
            {
                check_new_args_count(this, new_args);
                return make_shared<Result>(new_args.at(0));
            }

            // ---------------------------------------------------------------- Constant
            void Constant::init(const element::Type& type, const Shape& shape)
            {
                NGRAPH_CHECK(type.is_static(), "Constant needs a static element type");
                set_output_type(0, type, shape);
                m_data.assign(shape_size(shape) * type.size(), 0);
            }

            Constant::Constant(const element::Type& type, const Shape& shape, const void* data)
            {
                init(type, shape);
                if (!m_data.empty())
                    memcpy(m_data.data(), data, m_data.size());
            }

            template <typename T>
            static void fill_as(vector<uint8_t>& bytes, const vector<double>& values, size_t n)
            {
                T* p = reinterpret_cast<T*>(bytes.data());
                for (size_t i = 0; i < n; ++i)
                    p[i] = static_cast<T>(values.size() == 1 ? values[0] : values[i]);
            }

            void Constant::fill(const vector<double>& values)
            {
                const size_t n = shape_size(get_output_shape(0));
                switch (get_output_element_type(0).get_type_enum())
                {
                case element::Type_t::boolean: fill_as<char>(m_data, values, n); break;
                case element::Type_t::f32: fill_as<float>(m_data, values, n); break;
                case element::Type_t::f64: fill_as<double>(m_data, values, n); break;
                case element::Type_t::i8: fill_as<int8_t>(m_data, values, n); break;
                case element::Type_t::i32: fill_as<int32_t>(m_data, values, n); break;
                case element::Type_t::i64: fill_as<int64_t>(m_data, values, n); break;
                case element::Type_t::u8: fill_as<uint8_t>(m_data, values, n); break;
                default: throw ngraph_error("unsupported Constant element type");
                }
            }

            vector<double> Constant::get_values_as_double() const
            {
                const size_t n = shape_size(get_output_shape(0));
                vector<double> v(n);
                for (size_t i = 0; i < n; ++i)
                {
                    switch (get_output_element_type(0).get_type_enum())
                    {
                    case element::Type_t::boolean: v[i] = get_data_ptr<char>()[i]; break;
                    case element::Type_t::f32: v[i] = get_data_ptr<float>()[i]; break;
                    case element::Type_t::f64: v[i] = get_data_ptr<double>()[i]; break;
                    case element::Type_t::i8: v[i] = get_data_ptr<int8_t>()[i]; break;
                    case element::Type_t::i32: v[i] = get_data_ptr<int32_t>()[i]; break;
                    case element::Type_t::i64: v[i] = static_cast<double>(get_data_ptr<int64_t>()[i]); break;
                    case element::Type_t::u8: v[i] = get_data_ptr<uint8_t>()[i]; break;
                    default: throw ngraph_error("unsupported Constant element type");
                    }
                }
                return v;
            }

            shared_ptr<Node> Constant::clone_with_new_inputs(const OutputVector& new_args) const
            {
                check_new_args_count(this, new_args);
                return make_shared<Constant>(get_output_element_type(0), get_output_shape(0), get_data_ptr());
            }

            // ---------------------------------------------------------------- unary / shape glue
            constexpr NodeTypeInfo Abs::type_info;
            Abs::Abs(const Output<Node>& arg) : Op({arg}) { constructor_validate_and_infer_types(); }
            void Abs::validate_and_infer_types() { set_output_type(0, get_input_element_type(0), get_input_shape(0)); }
            shared_ptr<Node> Abs::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Abs>(a.at(0));
            }

            constexpr NodeTypeInfo Relu::type_info;
            Relu::Relu(const Output<Node>& arg) : Op({arg}) { constructor_validate_and_infer_types(); }
            void Relu::validate_and_infer_types() { set_output_type(0, get_input_element_type(0), get_input_shape(0)); }
            shared_ptr<Node> Relu::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Relu>(a.at(0));
            }

            constexpr NodeTypeInfo Convert::type_info;
            Convert::Convert(const Output<Node>& arg, const element::Type& t) : Op({arg}), m_type(t) { constructor_validate_and_infer_types(); }
            void Convert::validate_and_infer_types() { set_output_type(0, m_type, get_input_shape(0)); }
            shared_ptr<Node> Convert::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Convert>(a.at(0), m_type);
            }

            constexpr NodeTypeInfo Broadcast::type_info;
            Broadcast::Broadcast(const Output<Node>& arg, const Shape& shape, const AxisSet& axes) : Op({arg}), m_shape(shape), m_axes(axes)
            {
                constructor_validate_and_infer_types();
            }
            void Broadcast::validate_and_infer_types()
            {
                for (size_t a : m_axes)
                    NODE_VALIDATION_CHECK(this, a < m_shape.size(), "Broadcast axis index (", a, ") exceeds specified output shape rank (broadcast axes: ", m_axes, ", output shape: ", m_shape, ").");
                Shape required;
                for (size_t i = 0; i < m_shape.size(); ++i)
                    if (!m_axes.count(i))
                        required.push_back(m_shape[i]);
                NODE_VALIDATION_CHECK(this,
                                      get_input_shape(0) == required,
                                      "Broadcast argument shape, specified output shape, and axes are incompatible (argument shape: ",
                                      get_input_shape(0),
                                      ", output shape: ",
                                      m_shape,
                                      ", broadcast axes: ",
                                      m_axes,
                                      ").");
                set_output_type(0, get_input_element_type(0), m_shape);
            }
            shared_ptr<Node> Broadcast::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Broadcast>(a.at(0), m_shape, m_axes);
            }

            constexpr NodeTypeInfo Reshape::type_info;
            Reshape::Reshape(const Output<Node>& arg, const AxisVector& order, const Shape& shape) : Op({arg}), m_order(order), m_shape(shape)
            {
                constructor_validate_and_infer_types();
            }
            void Reshape::validate_and_infer_types()
            {
                const Shape& in = get_input_shape(0);
                NODE_VALIDATION_CHECK(this, m_order.size() == in.size(), "Input axis order is not a permutation of argument's axis indices (axis order: ", m_order.size(), " entries, argument shape: ", in, ").");
                vector<bool> seen(in.size(), false);
                for (size_t a : m_order)
                {
                    NODE_VALIDATION_CHECK(this, a < in.size() && !seen[a], "Input axis order is not a permutation of argument's axis indices (argument shape: ", in, ").");
                    seen[a] = true;
                }
                NODE_VALIDATION_CHECK(this,
                                      shape_size(in) == shape_size(m_shape),
                                      "Product of output shape dimensions does not match product of argument shape dimensions (output shape: ",
                                      m_shape,
                                      ", argument shape: ",
                                      in,
                                      ").");
                set_output_type(0, get_input_element_type(0), m_shape);
            }
            bool Reshape::get_is_transpose() const
            {
                for (size_t i = 0; i < m_order.size(); ++i)
                    if (m_order[i] != i)
                        return true;
                return false;
            }
            shared_ptr<Node> Reshape::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Reshape>(a.at(0), m_order, m_shape);
            }

            // ---------------------------------------------------------------- Quantize / Dequantize
            static Shape project_shape(const Shape& s, const AxisSet& axes)
            {
                Shape r;
                for (size_t i = 0; i < s.size(); ++i)
                    if (axes.count(i))
                        r.push_back(s[i]);
                return r;
            }

            constexpr NodeTypeInfo Quantize::type_info;
            Quantize::Quantize(const Output<Node>& input,
                               const Output<Node>& scale,
                               const Output<Node>& zero_point,
                               const element::Type& type,
                               const AxisSet& axes,
                               RoundMode round_mode)
                : Op({input, scale, zero_point}), m_type(type), m_axes(axes), m_round_mode(round_mode)
            {
                constructor_validate_and_infer_types();
            }

            void Quantize::validate_and_infer_types()
            {
                enum { INPUT, SCALE, ZERO_POINT };
                NODE_VALIDATION_CHECK(this, m_type.is_static(), "Output element type must not be dynamic");
                NODE_VALIDATION_CHECK(this, m_type.is_quantized(), "Output element type (", m_type, ") must be a quantized type");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(INPUT).compatible(get_input_element_type(SCALE)),
                                      "Scale element type (",
                                      get_input_element_type(SCALE),
                                      ") must match input element type (",
                                      get_input_element_type(INPUT),
                                      ")");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(INPUT).is_dynamic() || get_input_element_type(INPUT).is_real(),
                                      "Scale / input element type (",
                                      get_input_element_type(INPUT),
                                      ") must be a floating point number");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(ZERO_POINT).compatible(m_type),
                                      "Zero point element type (",
                                      get_input_element_type(ZERO_POINT),
                                      ") must match output element type (",
                                      m_type,
                                      ")");
                const Shape& input_shape = get_input_shape(INPUT);
                for (size_t axis : m_axes)
                    NODE_VALIDATION_CHECK(this, axis < input_shape.size(), "Quantization axis (", axis, ") must be less than input shape rank (", input_shape.size(), ")");
                NODE_VALIDATION_CHECK(this,
                                      get_input_shape(SCALE) == get_input_shape(ZERO_POINT),
                                      "Scale shape (",
                                      get_input_shape(SCALE),
                                      ") and zero point shape (",
                                      get_input_shape(ZERO_POINT),
                                      ") must match");
                NODE_VALIDATION_CHECK(this,
                                      get_input_shape(SCALE).size() == m_axes.size(),
                                      "Scale / zero point rank (",
                                      get_input_shape(SCALE).size(),
                                      ") does not match the number of quantization axes (",
                                      m_axes.size(),
                                      ")");
                NODE_VALIDATION_CHECK(this,
                                      get_input_shape(SCALE) == project_shape(input_shape, m_axes),
                                      "Scale / zero point shape (",
                                      get_input_shape(SCALE),
                                      ") must match input shape (",
                                      input_shape,
                                      ") at the quantization axes (",
                                      m_axes,
                                      ")");
                set_output_type(0, m_type, input_shape);
            }

            shared_ptr<Node> Quantize::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Quantize>(a.at(0), a.at(1), a.at(2), m_type, m_axes, m_round_mode);
            }

            constexpr NodeTypeInfo Dequantize::type_info;
            Dequantize::Dequantize(const Output<Node>& input,
                                   const Output<Node>& scale,
                                   const Output<Node>& zero_point,
                                   const element::Type& type,
                                   const AxisSet& axes)
                : Op({input, scale, zero_point}), m_type(type), m_axes(axes)
            {
                constructor_validate_and_infer_types();
            }

            void Dequantize::validate_and_infer_types()
            {
                enum { INPUT, SCALE, ZERO_POINT };
                NODE_VALIDATION_CHECK(this, m_type.is_static(), "Output element type must not be dynamic");
                NODE_VALIDATION_CHECK(this, m_type.is_real(), "Output element type (", m_type, ") must be a floating point type");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(INPUT).compatible(get_input_element_type(ZERO_POINT)),
                                      "Zero point element type (",
                                      get_input_element_type(ZERO_POINT),
                                      ") must match input element type (",
                                      get_input_element_type(INPUT),
                                      ")");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(INPUT).is_dynamic() || get_input_element_type(INPUT).is_quantized(),
                                      "Zero point / input element type (",
                                      get_input_element_type(INPUT),
                                      ") must be a quantized type");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(SCALE).compatible(m_type),
                                      "Scale element type (",
                                      get_input_element_type(SCALE),
                                      ") must match output element type (",
                                      m_type,
                                      ")");
                const Shape& input_shape = get_input_shape(INPUT);
                for (size_t axis : m_axes)
                    NODE_VALIDATION_CHECK(this, axis < input_shape.size(), "Quantization axis (", axis, ") must be less than input shape rank (", input_shape.size(), ")");
                NODE_VALIDATION_CHECK(this,
                                      get_input_shape(SCALE) == get_input_shape(ZERO_POINT),
                                      "Scale shape (",
                                      get_input_shape(SCALE),
                                      ") and zero point shape (",
                                      get_input_shape(ZERO_POINT),
                                      ") must match");
                NODE_VALIDATION_CHECK(this,
                                      get_input_shape(SCALE).size() == m_axes.size(),
                                      "Scale / zero point rank (",
                                      get_input_shape(SCALE).size(),
                                      ") does not match the number of quantization axes (",
                                      m_axes.size(),
                                      ")");
                NODE_VALIDATION_CHECK(this,
                                      get_input_shape(SCALE) == project_shape(input_shape, m_axes),
                                      "Scale / zero point shape (",
                                      get_input_shape(SCALE),
                                      ") must match input shape (",
                                      input_shape,
                                      ") at the quantization axes (",
                                      m_axes,
                                      ")");
                set_output_type(0, m_type, input_shape);
            }

            shared_ptr<Node> Dequantize::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Dequantize>(a.at(0), a.at(1), a.at(2), m_type, m_axes);
            }

            // ---------------------------------------------------------------- QuantizedConvolution
            constexpr NodeTypeInfo QuantizedConvolution::type_info;
            QuantizedConvolution::QuantizedConvolution(const Output<Node>& input,
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
                                                       const AxisSet& input_axes,
                                                       const AxisSet& filter_axes,
                                                       const AxisSet& output_axes)
                : Op({input, filters, input_scale, input_zero_point, filter_scale, filter_zero_point, output_scale, output_zero_point})
                , ConvAttributes(window_movement_strides, window_dilation_strides, padding_below, padding_above, data_dilation_strides)
                , m_output_type(output_type)
                , m_input_axes(input_axes)
                , m_filter_axes(filter_axes)
                , m_output_axes(output_axes)
            {
                constructor_validate_and_infer_types();
            }

            void QuantizedConvolution::validate_and_infer_types()
            {
                enum { INPUT, FILTER, INPUT_SCALE, INPUT_ZERO_POINT, FILTER_SCALE, FILTER_ZERO_POINT, OUTPUT_SCALE, OUTPUT_ZERO_POINT };
                NODE_VALIDATION_CHECK(this, m_output_type.is_static(), "Output element type must not be dynamic");
                NODE_VALIDATION_CHECK(this, m_output_type.is_quantized(), "Output element type (", m_output_type, ") must be a quantized type");
                NODE_VALIDATION_CHECK(this, get_input_element_type(INPUT).is_quantized(), "Input element type (", get_input_element_type(INPUT), ") must be a quantized type");
                NODE_VALIDATION_CHECK(this, get_input_element_type(FILTER).is_quantized(), "Filter element type (", get_input_element_type(FILTER), ") must be a quantized type");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(INPUT_SCALE).is_real() || get_input_element_type(FILTER_SCALE).is_real() ||
                                          get_input_element_type(OUTPUT_SCALE).is_real(),
                                      "Scale must be a floating point number");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(INPUT).compatible(get_input_element_type(INPUT_ZERO_POINT)),
                                      "Input Zero point element type (",
                                      get_input_element_type(INPUT_ZERO_POINT),
                                      ") must match input element type (",
                                      get_input_element_type(INPUT),
                                      ")");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(FILTER).compatible(get_input_element_type(FILTER_ZERO_POINT)),
                                      "Filter Zero point element type (",
                                      get_input_element_type(FILTER_ZERO_POINT),
                                      ") must match filter element type (",
                                      get_input_element_type(FILTER),
                                      ")");
                // scalar scales and zero points only (quantized_convolution.cpp:126-146)
                NODE_VALIDATION_CHECK(this, get_input_shape(2).empty() && get_input_shape(3).empty(), "Input scale and input zero point shape must be same and 1");
                NODE_VALIDATION_CHECK(this, get_input_shape(4).empty() && get_input_shape(5).empty(), "Filter scale and filter zero point shape must be same and 1");
                NODE_VALIDATION_CHECK(this, get_input_shape(6).empty() && get_input_shape(7).empty(), "Output scale and output zero point shape must be same and 1");
                NODE_VALIDATION_CHECK(this,
                                      m_input_axes.empty() && m_filter_axes.empty() && m_output_axes.empty(),
                                      "Input, filter and output AxisSet should be empty");
                Shape result_shape = infer_convolution_forward(this,
                                                               get_input_shape(INPUT),
                                                               m_data_dilation_strides,
                                                               m_padding_below,
                                                               m_padding_above,
                                                               get_input_shape(FILTER),
                                                               m_window_movement_strides,
                                                               m_window_dilation_strides);
                NODE_VALIDATION_CHECK(this,
                                      m_output_type.compatible(get_input_element_type(OUTPUT_ZERO_POINT)),
                                      "Output Zero point element type (",
                                      get_input_element_type(OUTPUT_ZERO_POINT),
                                      ") must match output element type (",
                                      m_output_type,
                                      ")");
                set_output_type(0, m_output_type, result_shape);
            }

            shared_ptr<Node> QuantizedConvolution::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<QuantizedConvolution>(a.at(0), a.at(1), m_window_movement_strides, m_window_dilation_strides, m_padding_below,
                                                         m_padding_above, m_data_dilation_strides, a.at(2), a.at(3), a.at(4), a.at(5), a.at(6),
                                                         a.at(7), m_output_type, m_input_axes, m_filter_axes, m_output_axes);
            }

            // ---------------------------------------------------------------- fused convolutions
            static Shape fused_conv_shape(const Node* n, const ConvAttributes& c, const Output<Node>& data, const Output<Node>& filters)
            {
                return infer_convolution_forward(n, data.get_shape(), c.get_data_dilation_strides(), c.get_padding_below(), c.get_padding_above(),
                                                 filters.get_shape(), c.get_window_movement_strides(), c.get_window_dilation_strides());
            }

            constexpr NodeTypeInfo QuantizedConvolutionBias::type_info;
            QuantizedConvolutionBias::QuantizedConvolutionBias(const Output<Node>& data_batch,
                                                               const Output<Node>& filters,
                                                               const Output<Node>& bias,
                                                               const Strides& s,
                                                               const Strides& d,
                                                               const CoordinateDiff& pb,
                                                               const CoordinateDiff& pa,
                                                               const Strides& dd,
                                                               const Output<Node>& scale,
                                                               const bool with_relu)
                : Op({data_batch, filters, bias, scale}), ConvAttributes(s, d, pb, pa, dd), m_with_relu(with_relu)
            {
                // quantized_conv_bias.cpp:52: u8 with relu, i8 otherwise
                set_output_type(0, with_relu ? element::u8 : element::i8, fused_conv_shape(this, *this, data_batch, filters));
            }
            shared_ptr<Node> QuantizedConvolutionBias::clone_with_new_inputs(const OutputVector& a) const
            {
                if (a.size() != 4)
                    throw ngraph_error("Incorrect number of new arguments");
                return make_shared<QuantizedConvolutionBias>(a.at(0), a.at(1), a.at(2), m_window_movement_strides, m_window_dilation_strides,
                                                             m_padding_below, m_padding_above, m_data_dilation_strides, a.at(3), m_with_relu);
            }

            constexpr NodeTypeInfo QuantizedConvolutionRelu::type_info;
            QuantizedConvolutionRelu::QuantizedConvolutionRelu(const Output<Node>& data_batch,
                                                               const Output<Node>& filters,
                                                               const Strides& s,
                                                               const Strides& d,
                                                               const CoordinateDiff& pb,
                                                               const CoordinateDiff& pa,
                                                               const Strides& dd,
                                                               const Output<Node>& scale)
                : Op({data_batch, filters, scale}), ConvAttributes(s, d, pb, pa, dd)
            {
                set_output_type(0, element::u8, fused_conv_shape(this, *this, data_batch, filters));
            }
            shared_ptr<Node> QuantizedConvolutionRelu::clone_with_new_inputs(const OutputVector& a) const
            {
                if (a.size() != 3)
                    throw ngraph_error("Incorrect number of new arguments");
                return make_shared<QuantizedConvolutionRelu>(a.at(0), a.at(1), m_window_movement_strides, m_window_dilation_strides,
                                                             m_padding_below, m_padding_above, m_data_dilation_strides, a.at(2));
            }

            constexpr NodeTypeInfo QuantizedConvolutionBiasAdd::type_info;
            QuantizedConvolutionBiasAdd::QuantizedConvolutionBiasAdd(const Output<Node>& data_batch,
                                                                     const Output<Node>& filters,
                                                                     const Output<Node>& bias,
                                                                     const Output<Node>& sum_input,
                                                                     const Strides& s,
                                                                     const Strides& d,
                                                                     const CoordinateDiff& pb,
                                                                     const CoordinateDiff& pa,
                                                                     const Strides& dd,
                                                                     const Output<Node>& scale,
                                                                     const Output<Node>& sum_scale,
                                                                     const bool with_relu)
                : Op({data_batch, filters, bias, sum_input, scale, sum_scale}), ConvAttributes(s, d, pb, pa, dd), m_with_relu(with_relu)
            {
                set_output_type(0, with_relu ? element::u8 : element::i8, fused_conv_shape(this, *this, data_batch, filters));
            }
            shared_ptr<Node> QuantizedConvolutionBiasAdd::clone_with_new_inputs(const OutputVector& a) const
            {
                if (a.size() != 6)
                    throw ngraph_error("Incorrect number of new arguments");
                return make_shared<QuantizedConvolutionBiasAdd>(a.at(0), a.at(1), a.at(2), a.at(3), m_window_movement_strides,
                                                                m_window_dilation_strides, m_padding_below, m_padding_above,
                                                                m_data_dilation_strides, a.at(4), a.at(5), m_with_relu);
            }

            constexpr NodeTypeInfo QuantizedConvolutionBiasSignedAdd::type_info;
            QuantizedConvolutionBiasSignedAdd::QuantizedConvolutionBiasSignedAdd(const Output<Node>& data_batch,
                                                                                 const Output<Node>& filters,
                                                                                 const Output<Node>& bias,
                                                                                 const Output<Node>& sum_input,
                                                                                 const Strides& s,
                                                                                 const Strides& d,
                                                                                 const CoordinateDiff& pb,
                                                                                 const CoordinateDiff& pa,
                                                                                 const Strides& dd,
                                                                                 const Output<Node>& scale,
                                                                                 const Output<Node>& sum_scale,
                                                                                 const bool with_relu)
                : Op({data_batch, filters, bias, sum_input, scale, sum_scale}), ConvAttributes(s, d, pb, pa, dd), m_with_relu(with_relu)
            {
                // quantized_conv_bias.cpp:197-199: the signed variant stays i8
                set_output_type(0, element::i8, fused_conv_shape(this, *this, data_batch, filters));
            }
            shared_ptr<Node> QuantizedConvolutionBiasSignedAdd::clone_with_new_inputs(const OutputVector& a) const
            {
                if (a.size() != 6)
                    throw ngraph_error("Incorrect number of new arguments");
                return make_shared<QuantizedConvolutionBiasSignedAdd>(a.at(0), a.at(1), a.at(2), a.at(3), m_window_movement_strides,
                                                                      m_window_dilation_strides, m_padding_below, m_padding_above,
                                                                      m_data_dilation_strides, a.at(4), a.at(5), m_with_relu);
            }

            // ---------------------------------------------------------------- dots
            constexpr NodeTypeInfo QuantizedDot::type_info;
            QuantizedDot::QuantizedDot(const Output<Node>& input0,
                                       const Output<Node>& input1,
                                       size_t reduction_axes_count,
                                       const Output<Node>& input0_scale,
                                       const Output<Node>& input0_zero_point,
                                       const Output<Node>& input1_scale,
                                       const Output<Node>& input1_zero_point,
                                       const Output<Node>& output_scale,
                                       const Output<Node>& output_zero_point,
                                       const element::Type& output_type,
                                       const AxisSet& input0_axes,
                                       const AxisSet& input1_axes,
                                       const AxisSet& output_axes)
                : Op({input0, input1, input0_scale, input0_zero_point, input1_scale, input1_zero_point, output_scale, output_zero_point})
                , m_reduction_axes_count(reduction_axes_count)
                , m_output_type(output_type)
                , m_input0_axes(input0_axes)
                , m_input1_axes(input1_axes)
                , m_output_axes(output_axes)
            {
                constructor_validate_and_infer_types();
            }

            void QuantizedDot::validate_and_infer_types()
            {
                enum { INPUT0, INPUT1, INPUT0_SCALE, INPUT0_ZERO_POINT, INPUT1_SCALE, INPUT1_ZERO_POINT, OUTPUT_SCALE, OUTPUT_ZERO_POINT };
                NODE_VALIDATION_CHECK(this, m_output_type.is_static(), "Output element type must not be dynamic");
                NODE_VALIDATION_CHECK(this, m_output_type.is_quantized(), "Output element type (", m_output_type, ") must be a quantized type");
                NODE_VALIDATION_CHECK(this, get_input_element_type(INPUT0).is_quantized(), "Input0 element type (", get_input_element_type(INPUT0), ") must be a quantized type");
                NODE_VALIDATION_CHECK(this, get_input_element_type(INPUT1).is_quantized(), "Input1 element type (", get_input_element_type(INPUT1), ") must be a quantized type");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(INPUT0_SCALE).is_real() || get_input_element_type(INPUT1_SCALE).is_real() ||
                                          get_input_element_type(OUTPUT_SCALE).is_real(),
                                      "Scale must be a floating point number");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(INPUT0).compatible(get_input_element_type(INPUT0_ZERO_POINT)),
                                      "Input0 Zero point element type (",
                                      get_input_element_type(INPUT0_ZERO_POINT),
                                      ") must match input0 element type (",
                                      get_input_element_type(INPUT0),
                                      ")");
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(INPUT1).compatible(get_input_element_type(INPUT1_ZERO_POINT)),
                                      "Input1 Zero point element type (",
                                      get_input_element_type(INPUT1_ZERO_POINT),
                                      ") must match input1 element type (",
                                      get_input_element_type(INPUT1),
                                      ")");
                NODE_VALIDATION_CHECK(this, get_input_shape(2).empty() && get_input_shape(3).empty(), "Input0 scale and input0 zero point shape must be same and 1");
                NODE_VALIDATION_CHECK(this, get_input_shape(4).empty() && get_input_shape(5).empty(), "Input1 scale and input1 zero point shape must be same and 1");
                NODE_VALIDATION_CHECK(this, get_input_shape(6).empty() && get_input_shape(7).empty(), "Output scale and output zero point shape must be same and 1");
                NODE_VALIDATION_CHECK(this,
                                      m_input0_axes.empty() && m_input1_axes.empty() && m_output_axes.empty(),
                                      "Input0, input1 and output AxisSet should be empty");
                const Shape& s0 = get_input_shape(INPUT0);
                const Shape& s1 = get_input_shape(INPUT1);
                NODE_VALIDATION_CHECK(this,
                                      m_reduction_axes_count <= s0.size() && m_reduction_axes_count <= s1.size(),
                                      "Reduction axes count (",
                                      m_reduction_axes_count,
                                      ") is too large (arg0 shape: ",
                                      s0,
                                      ", arg1 shape: ",
                                      s1,
                                      ").");
                for (size_t i = 0; i < m_reduction_axes_count; ++i)
                {
                    size_t a0 = s0.size() - m_reduction_axes_count + i;
                    NODE_VALIDATION_CHECK(this,
                                          s0[a0] == s1[i],
                                          "Paired axes (axis ",
                                          a0,
                                          " from arg0, axis ",
                                          i,
                                          " from arg1) do not have same length (arg0 shape: ",
                                          s0,
                                          ", arg1 shape: ",
                                          s1,
                                          ", reduction axes count: ",
                                          m_reduction_axes_count,
                                          ").");
                }
                Shape result;
                for (size_t j = 0; j + m_reduction_axes_count < s0.size(); ++j)
                    result.push_back(s0[j]);
                for (size_t j = m_reduction_axes_count; j < s1.size(); ++j)
                    result.push_back(s1[j]);
                NODE_VALIDATION_CHECK(this,
                                      m_output_type.compatible(get_input_element_type(OUTPUT_ZERO_POINT)),
                                      "Output Zero point element type (",
                                      get_input_element_type(OUTPUT_ZERO_POINT),
                                      ") must match output element type (",
                                      m_output_type,
                                      ")");
                set_output_type(0, m_output_type, result);
            }

            shared_ptr<Node> QuantizedDot::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<QuantizedDot>(a.at(0), a.at(1), m_reduction_axes_count, a.at(2), a.at(3), a.at(4), a.at(5), a.at(6), a.at(7),
                                                 m_output_type, m_input0_axes, m_input1_axes, m_output_axes);
            }

            constexpr NodeTypeInfo QuantizedDotBias::type_info;
            QuantizedDotBias::QuantizedDotBias(const Output<Node>& data,
                                               const Output<Node>& weights,
                                               const Output<Node>& bias,
                                               const Output<Node>& scale,
                                               bool requantize,
                                               bool with_relu)
                : Op({data, weights, bias, scale}), m_requantize(requantize), m_with_relu(with_relu)
            {
                const Shape& ds = data.get_shape();
                const Shape& ws = weights.get_shape();
                const Shape& bs = bias.get_shape();
                NODE_VALIDATION_CHECK(this, ds.size() == 2 && ws.size() == 2 && ds[1] == ws[1], "only valid tensors of rank 2 supported. data ", ds, " weights ", ws);
                NODE_VALIDATION_CHECK(this, bs.size() == 1 && bs[0] == ws[0], "invalid bias ", bs);
                // quantized_dot_bias.cpp:54
                auto et = requantize ? (with_relu ? element::u8 : element::i8) : element::f32;
                set_output_type(0, et, Shape{ds[0], ws[0]});
            }
            shared_ptr<Node> QuantizedDotBias::clone_with_new_inputs(const OutputVector& a) const
            {
                if (a.size() != 4)
                    throw ngraph_error("Incorrect number of new arguments");
                return make_shared<QuantizedDotBias>(a.at(0), a.at(1), a.at(2), a.at(3), m_requantize, m_with_relu);
            }

            // ---------------------------------------------------------------- pooling
            static Shape pool_shape(const Node* n, const Shape& in, const Shape& window, const Strides& strides, const Shape& pb, const Shape& pa)
            {
                NODE_VALIDATION_CHECK(n, in.size() >= 3, "Data batch must have rank of at least 3 (data batch shape: ", in, ").");
                const size_t ns = in.size() - 2;
                NODE_VALIDATION_CHECK(n,
                                      window.size() == ns && strides.size() == ns && pb.size() == ns && pa.size() == ns,
                                      "Ranks for data item shape (data batch has shape ",
                                      in,
                                      "), padding below, padding above, window shape and window strides do not match.");
                Shape out{in[0], in[1]};
                for (size_t i = 0; i < ns; ++i)
                {
                    NODE_VALIDATION_CHECK(n, window[i] > 0 && strides[i] > 0, "Window shape / strides have a zero dimension at axis ", i, ".");
                    size_t padded = in[2 + i] + pb[i] + pa[i];
                    NODE_VALIDATION_CHECK(n, window[i] <= padded, "Window after dilation has dimension (dim: ", window[i], ") larger than the data shape after padding (dim: ", padded, ") at axis ", i, ".");
                    out.push_back((padded - window[i]) / strides[i] + 1);
                }
                return out;
            }

            constexpr NodeTypeInfo MaxPool::type_info;
            MaxPool::MaxPool(const Output<Node>& arg, const Shape& window, const Strides& strides, const Shape& pb, const Shape& pa)
                : Op({arg}), m_window_shape(window), m_strides(strides), m_padding_below(pb), m_padding_above(pa)
            {
                constructor_validate_and_infer_types();
            }
            void MaxPool::validate_and_infer_types()
            {
                set_output_type(0, get_input_element_type(0), pool_shape(this, get_input_shape(0), m_window_shape, m_strides, m_padding_below, m_padding_above));
            }
            shared_ptr<Node> MaxPool::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<MaxPool>(a.at(0), m_window_shape, m_strides, m_padding_below, m_padding_above);
            }

            constexpr NodeTypeInfo AvgPool::type_info;
            AvgPool::AvgPool(const Output<Node>& arg, const Shape& window, const Strides& strides, const Shape& pb, const Shape& pa, bool include_padding)
                : Op({arg}), m_window_shape(window), m_strides(strides), m_padding_below(pb), m_padding_above(pa), m_include_padding(include_padding)
            {
                constructor_validate_and_infer_types();
            }
            void AvgPool::validate_and_infer_types()
            {
                set_output_type(0, get_input_element_type(0), pool_shape(this, get_input_shape(0), m_window_shape, m_strides, m_padding_below, m_padding_above));
            }
            shared_ptr<Node> AvgPool::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<AvgPool>(a.at(0), m_window_shape, m_strides, m_padding_below, m_padding_above, m_include_padding);
            }

            // ---- fp32 glue of a transformer encoder --------------------------------------------------
            constexpr NodeTypeInfo Softmax::type_info;
            Softmax::Softmax(const Output<Node>& arg, const AxisSet& axes) : Op({arg}), m_axes(axes) { constructor_validate_and_infer_types(); }
            void Softmax::validate_and_infer_types()
            {
                // src/ngraph/op/softmax.cpp:56-70; an empty set means every axis (:45-52)
                const Shape& s = get_input_shape(0);
                if (m_axes.empty())
                    for (size_t i = 0; i < s.size(); ++i)
                        m_axes.insert(i);
                for (auto axis : m_axes)
                    NODE_VALIDATION_CHECK(this, axis < s.size(), "Reduction axis (", axis, ") is out of bounds (argument shape: ", s, ").");
                set_output_type(0, get_input_element_type(0), s);
            }
            shared_ptr<Node> Softmax::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Softmax>(a.at(0), m_axes);
            }

            constexpr NodeTypeInfo Erf::type_info;
            Erf::Erf(const Output<Node>& arg) : Op({arg}) { constructor_validate_and_infer_types(); }
            void Erf::validate_and_infer_types() { set_output_type(0, get_input_element_type(0), get_input_shape(0)); }
            shared_ptr<Node> Erf::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Erf>(a.at(0));
            }

            constexpr NodeTypeInfo Gelu::type_info;
            Gelu::Gelu(const Output<Node>& arg) : Op({arg}) { constructor_validate_and_infer_types(); }
            void Gelu::validate_and_infer_types()
            {
                // src/ngraph/op/gelu.cpp:71-90
                NODE_VALIDATION_CHECK(this, get_input_element_type(0).is_real(), "Argument element type must be f16, bf16, f32, f64 or dynamic (got ", get_input_element_type(0), ").");
                set_output_type(0, get_input_element_type(0), get_input_shape(0));
            }
            shared_ptr<Node> Gelu::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Gelu>(a.at(0));
            }

            constexpr NodeTypeInfo LayerNorm::type_info;
            LayerNorm::LayerNorm(const Output<Node>& data, const Output<Node>& scale, const Output<Node>& bias, bool keep_stats, int64_t begin_norm_axis, double epsilon)
                : Op({data, scale, bias}), m_keep_stats(keep_stats), m_use_affine(true), m_begin_norm_axis(begin_norm_axis), m_epsilon(epsilon)
            {
                constructor_validate_and_infer_types();
            }
            LayerNorm::LayerNorm(const Output<Node>& data, bool keep_stats, int64_t begin_norm_axis, double epsilon)
                : Op({data}), m_keep_stats(keep_stats), m_use_affine(false), m_begin_norm_axis(begin_norm_axis), m_epsilon(epsilon)
            {
                constructor_validate_and_infer_types();
            }
            void LayerNorm::validate_and_infer_types()
            {
                // src/ngraph/op/layer_norm.cpp:173-235, static shapes
                const element::Type& et = get_input_element_type(0);
                NODE_VALIDATION_CHECK(this, et.is_real(), "Argument element type must be f16, bf16, f32, f64 or dynamic (got ", et, ").");
                const Shape& ds = get_input_shape(0);
                const int64_t d_rank = static_cast<int64_t>(ds.size());
                const int64_t n_axis = m_begin_norm_axis >= 0 ? m_begin_norm_axis : d_rank + m_begin_norm_axis;
                NODE_VALIDATION_CHECK(this, n_axis >= 0 && n_axis < d_rank, "begin_norm_axis is out of range");
                if (m_use_affine)
                {
                    const int64_t s_rank = static_cast<int64_t>(get_input_shape(1).size()), b_rank = static_cast<int64_t>(get_input_shape(2).size());
                    NODE_VALIDATION_CHECK(this, s_rank == b_rank && (s_rank == d_rank - n_axis || s_rank == 1), "Scale and/or bias rank is incorrect");
                }
                if (m_keep_stats)
                {
                    set_output_size(3);
                    const Shape stats(ds.begin(), ds.begin() + n_axis);
                    set_output_type(1, et, stats);
                    set_output_type(2, et, stats);
                }
                set_output_type(0, et, ds);
            }
            shared_ptr<Node> LayerNorm::clone_with_new_inputs(const OutputVector& a) const
            {
                // src/ngraph/op/layer_norm.cpp:148-170
                if (a.size() != 1 && a.size() != 3)
                    throw ngraph_error("Incorrect number of new arguments");
                if (!m_use_affine)
                    return make_shared<LayerNorm>(a.at(0), m_keep_stats, m_begin_norm_axis, m_epsilon);
                return make_shared<LayerNorm>(a.at(0), a.at(1), a.at(2), m_keep_stats, m_begin_norm_axis, m_epsilon);
            }

            namespace
            {
                // src/ngraph/op/experimental/batch_mat_mul.cpp:39-77 and batch_mat_mul_transpose.cpp:113-160
                Shape batch_mat_mul_shape(const Node* n, const char* name, bool t0, bool t1)
                {
                    NODE_VALIDATION_CHECK(n, n->get_input_element_type(0) == n->get_input_element_type(1), "Inputs arg0 and arg1 must have compatible element type.");
                    const Shape& a = n->get_input_shape(0);
                    const Shape& b = n->get_input_shape(1);
                    NODE_VALIDATION_CHECK(n, a.size() == 3, "Input arg0 shape must have rank 3, got ", a.size(), ".");
                    NODE_VALIDATION_CHECK(n, b.size() == 3, "Input arg1 shape must have rank 3, got ", b.size(), ".");
                    NODE_VALIDATION_CHECK(n, a[0] == b[0], "Batch size dimensions are not equal while creating ", name, ".");
                    const size_t m = t0 ? a[2] : a[1], k0 = t0 ? a[1] : a[2], k1 = t1 ? b[2] : b[1], nn = t1 ? b[1] : b[2];
                    NODE_VALIDATION_CHECK(n, k0 == k1, "Product dimensions are not equal while creating ", name, ".");
                    return Shape{a[0], m, nn};
                }
            }

            constexpr NodeTypeInfo BatchMatMul::type_info;
            BatchMatMul::BatchMatMul(const Output<Node>& arg0, const Output<Node>& arg1) : Op({arg0, arg1}) { constructor_validate_and_infer_types(); }
            void BatchMatMul::validate_and_infer_types() { set_output_type(0, get_input_element_type(0), batch_mat_mul_shape(this, "BatchMatMul", false, false)); }
            shared_ptr<Node> BatchMatMul::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<BatchMatMul>(a.at(0), a.at(1));
            }

            constexpr NodeTypeInfo BatchMatMulTranspose::type_info;
            BatchMatMulTranspose::BatchMatMulTranspose(const Output<Node>& arg0, const Output<Node>& arg1, bool t0, bool t1) : Op({arg0, arg1}), m_transpose_arg0(t0), m_transpose_arg1(t1)
            {
                constructor_validate_and_infer_types();
            }
            void BatchMatMulTranspose::validate_and_infer_types()
            {
                set_output_type(0, get_input_element_type(0), batch_mat_mul_shape(this, "BatchMatMulTranspose", m_transpose_arg0, m_transpose_arg1));
            }
            shared_ptr<Node> BatchMatMulTranspose::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<BatchMatMulTranspose>(a.at(0), a.at(1), m_transpose_arg0, m_transpose_arg1);
            }

            constexpr NodeTypeInfo Concat::type_info;
            Concat::Concat(const OutputVector& args, int64_t axis) : Op(args), m_axis(axis) { constructor_validate_and_infer_types(); }
            void Concat::validate_and_infer_types()
            {
                // src/ngraph/op/concat.cpp:42-100, static shapes only
                NODE_VALIDATION_CHECK(this, get_input_size() >= 1, "At least one argument required.");
                const int64_t rank = static_cast<int64_t>(get_input_shape(0).size());
                if (m_concat_axis < 0)
                    m_concat_axis = m_axis < 0 ? m_axis + rank : m_axis;
                Shape out = get_input_shape(0);
                size_t joined = 0;
                for (size_t i = 0; i < get_input_size(); ++i)
                {
                    NODE_VALIDATION_CHECK(this, get_input_element_type(i) == get_input_element_type(0), "Argument element types are inconsistent.");
                    const Shape& s = get_input_shape(i);
                    NODE_VALIDATION_CHECK(this,
                                          m_concat_axis >= 0 && m_concat_axis < static_cast<int64_t>(s.size()),
                                          "Concatenation axis (",
                                          m_concat_axis,
                                          ") is out of bounds for argument ",
                                          i,
                                          ", which has shape ",
                                          s,
                                          ".");
                    bool same = s.size() == out.size();
                    for (size_t a = 0; same && a < s.size(); ++a)
                        same = static_cast<int64_t>(a) == m_concat_axis || s[a] == out[a];
                    NODE_VALIDATION_CHECK(this,
                                          same,
                                          "Argument shapes are inconsistent; they must have the same rank, and must have equal dimension "
                                          "everywhere except on the concatenation axis (axis ",
                                          m_concat_axis,
                                          ").");
                    joined += s[m_concat_axis];
                }
                out[m_concat_axis] = joined;
                set_output_type(0, get_input_element_type(0), out);
            }
            shared_ptr<Node> Concat::clone_with_new_inputs(const OutputVector& a) const { return make_shared<Concat>(a, m_axis); }

            // src/ngraph/op/slice.cpp:25-128
            constexpr NodeTypeInfo Slice::type_info;
            Slice::Slice(const Output<Node>& arg, const Coordinate& lower_bounds, const Coordinate& upper_bounds, const Strides& strides)
                : Op({arg}), m_lower_bounds(lower_bounds), m_upper_bounds(upper_bounds), m_strides(strides)
            {
                constructor_validate_and_infer_types();
            }
            Slice::Slice(const Output<Node>& arg, const Coordinate& lower_bounds, const Coordinate& upper_bounds)
                : Op({arg}), m_lower_bounds(lower_bounds), m_upper_bounds(upper_bounds), m_strides(Strides())
            {
                constructor_validate_and_infer_types();
            }
            void Slice::validate_and_infer_types()
            {
                if (m_strides.size() == 0) // no strides given: ones
                    m_strides = Strides(m_lower_bounds.size(), 1);
                NODE_VALIDATION_CHECK(this,
                                      m_lower_bounds.size() == m_upper_bounds.size() && m_lower_bounds.size() == m_strides.size(),
                                      "Ranks of lower bounds (",
                                      m_lower_bounds,
                                      "), upper bounds (",
                                      m_upper_bounds,
                                      ") and strides (",
                                      m_strides,
                                      ") do not match.");
                const size_t output_rank = m_upper_bounds.size();
                for (size_t i = 0; i < output_rank; i++)
                {
                    NODE_VALIDATION_CHECK(this,
                                          m_lower_bounds[i] <= m_upper_bounds[i],
                                          "Lower bound for slice is greater than upper bound at axis ",
                                          i,
                                          " (lower bounds: ",
                                          m_lower_bounds,
                                          ", upper bounds: ",
                                          m_upper_bounds,
                                          ").");
                    NODE_VALIDATION_CHECK(this, m_strides[i] != 0, "Stride for slice is zero at axis ", i, " (strides: ", m_strides, ").");
                }
                const Shape& input_shape = get_input_shape(0);
                NODE_VALIDATION_CHECK(this,
                                      input_shape.size() == output_rank,
                                      "Input rank does not match the rank of the lower bounds (",
                                      m_lower_bounds,
                                      "), upper bounds (",
                                      m_upper_bounds,
                                      "), and strides (",
                                      m_strides,
                                      ").");
                Shape result(output_rank);
                for (size_t i = 0; i < output_rank; i++)
                {
                    NODE_VALIDATION_CHECK(this,
                                          m_upper_bounds[i] <= input_shape[i],
                                          "Upper bound for slice at axis ",
                                          i,
                                          " is out of range ",
                                          "(upper bounds: ",
                                          m_upper_bounds,
                                          ", argument shape: ",
                                          input_shape,
                                          ").");
                    const size_t extent = m_upper_bounds[i] - m_lower_bounds[i];
                    result[i] = extent / m_strides[i] + ((extent % m_strides[i] == 0) ? 0 : 1);
                }
                set_output_type(0, get_input_element_type(0), result);
            }
            shared_ptr<Node> Slice::clone_with_new_inputs(const OutputVector& a) const
            {
                check_new_args_count(this, a);
                return make_shared<Slice>(a.at(0), m_lower_bounds, m_upper_bounds, m_strides);
            }
        }

        namespace v1
        {
            constexpr NodeTypeInfo Add::type_info;
            constexpr NodeTypeInfo Subtract::type_info;
            constexpr NodeTypeInfo Multiply::type_info;
            constexpr NodeTypeInfo Divide::type_info;
            constexpr NodeTypeInfo Maximum::type_info;
            constexpr NodeTypeInfo Minimum::type_info;

            void BinaryElementwise::validate_and_infer_types()
            {
                NODE_VALIDATION_CHECK(this,
                                      get_input_element_type(0) == get_input_element_type(1),
                                      "Argument element types are inconsistent (",
                                      get_input_element_type(0),
                                      " vs ",
                                      get_input_element_type(1),
                                      ").");
                const Shape& a = get_input_shape(0);
                const Shape& b = get_input_shape(1);
                Shape out;
                if (a == b)
                    out = a;
                else if (shape_size(b) == 1 && b.size() <= a.size())
                    out = a;
                else if (shape_size(a) == 1 && a.size() <= b.size())
                    out = b;
                else
                    NODE_VALIDATION_CHECK(this, false, "Argument shapes are inconsistent (", a, " vs ", b, ").");
                set_output_type(0, get_input_element_type(0), out);
            }
        }
    }

    shared_ptr<Node> operator+(const Output<Node>& a, const Output<Node>& b) { return make_shared<op::v1::Add>(a, b); }
    shared_ptr<Node> operator-(const Output<Node>& a, const Output<Node>& b) { return make_shared<op::v1::Subtract>(a, b); }
    shared_ptr<Node> operator*(const Output<Node>& a, const Output<Node>& b) { return make_shared<op::v1::Multiply>(a, b); }
    shared_ptr<Node> operator/(const Output<Node>& a, const Output<Node>& b) { return make_shared<op::v1::Divide>(a, b); }
}
