// JSON form of a Function, as src/ngraph/serializer.hpp:26-63 of the nGraph tree declares it.
//
// The reader accepts what nGraph's JSONSerializer writes (src/ngraph/serializer.cpp:556-581 for a
// function, :2661-3700 for a node) for the ops of the int8 inference path and its glue: Parameter,
// Constant, Result, Quantize, Dequantize, QuantizedConvolution, QuantizedDot, Convert, Broadcast,
// Reshape, Abs, Relu, MaxPool, AvgPool, Concat, Softmax, Erf, Gelu, LayerNorm, BatchMatMul,
// BatchMatMulTranspose and the binary elementwise Add / Subtract / Multiply / Divide / Maximum /
// Minimum (opset-0 spelling and the attribute-visitor spelling of opset 1), plus the GetOutputElement
// alias of older files.  Any other op stops the reader with nGraph's own message,
// "Error parsing json at node '<name>'", followed by the reason.  The fused quantized ops
// (QuantizedConvolutionBias ..., QuantizedDotBias) have no JSON form in nGraph either
// (serializer.cpp:2117-2123, 2159): they come into being when the backend's fusion pass runs on the
// loaded graph.  cpio containers (Executable::save) are recognised and refused.
//
// The writer produces the same layout (keys sorted, as nlohmann::json's std::map does), so a graph
// written here loads in nGraph and the other way round.
#pragma once

#include <iosfwd>
#include <memory>
#include <string>

#include "ngraph/core.hpp"

namespace ngraph
{
    /// Serialize a Function to a json string; indent 0 is the compact form.
    NGRAPH_API std::string serialize(std::shared_ptr<ngraph::Function> func, size_t indent = 0);
    /// Serialize a Function to a json file.
    NGRAPH_API void serialize(const std::string& path, std::shared_ptr<ngraph::Function> func, size_t indent = 0);
    /// Serialize a Function to a stream.
    NGRAPH_API void serialize(std::ostream& out, std::shared_ptr<ngraph::Function> func, size_t indent = 0);
    /// Deserialize a Function from a stream.
    NGRAPH_API std::shared_ptr<ngraph::Function> deserialize(std::istream& in);
    /// Deserialize a Function from a json string, or from the file of that name if one exists.
    NGRAPH_API std::shared_ptr<ngraph::Function> deserialize(const std::string& str);
}
