// ONNX model ingress for the quantized path: the entry points of
// src/ngraph/frontend/onnx_import/onnx.hpp:43-82 of the nGraph tree, for the operators that end in
// the ops this library accelerates (QuantizeLinear, DequantizeLinear, QLinearConv, QLinearMatMul,
// ConvInteger, MatMulInteger) and the little glue their models carry (Constant, Identity, Relu,
// Add).  A model is read as binary protobuf or, failing that, as protobuf text (the reference tries
// the two in the same order, onnx.cpp:54-71); neither libprotobuf nor the ONNX schema is needed:
// the handful of messages involved is decoded by hand.
#pragma once

#include <cstdint>
#include <istream>
#include <memory>
#include <set>
#include <string>

#include "ngraph/core.hpp"

namespace ngraph
{
    namespace onnx_import
    {
        /// Operators of the given opset version and domain ("" or "ai.onnx") this importer maps.
        NGRAPH_API std::set<std::string> get_supported_operators(std::int64_t version, const std::string& domain);
        NGRAPH_API bool is_operator_supported(const std::string& op_name, std::int64_t version, const std::string& domain = "ai.onnx");

        /// Reads an ONNX model (binary or text protobuf) and builds the nGraph function: graph inputs
        /// that have no initializer become Parameters (in the graph's order), initializers become
        /// Constants, graph outputs the function's results.  Throws ngraph_error on a file that cannot
        /// be opened or parsed and on operators outside the set above.
        NGRAPH_API std::shared_ptr<Function> import_onnx_model(std::istream& stream);
        NGRAPH_API std::shared_ptr<Function> import_onnx_model(const std::string& file_path);
    }
}
