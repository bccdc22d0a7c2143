// Quantization-aware graph rewrites of the HIP backend: the counterpart of the reference CPU
// backend's CPUQuantFusion (src/ngraph/runtime/cpu/pass/cpu_fusion.hpp, cpu_fusion.cpp:2025-2609).
// Run by the backend on its private copy of a function before lowering; NGRAPH_PASS_ENABLES
// "HIPQuantFusion:0" switches it off.
#pragma once

#include "ngraph/pass/pass.hpp"

namespace ngraph
{
    namespace runtime
    {
        namespace hip
        {
            namespace pass
            {
                // Rewrites, each the reference's pattern of the same name:
                //   QConvRelu      Relu(Dequantize(QuantizedConvolution))      -> Dequantize(QuantizedConvolutionRelu)
                //   QConvBiasRelu  Relu(Dequantize(QuantizedConvolutionBias))  -> Dequantize(QuantizedConvolutionBias, with_relu)
                //   QConvBiasAdd   Relu(Dequantize(QuantizedConvolutionBias) + Dequantize(s)) -> Dequantize(QuantizedConvolutionBias[Signed]Add)
                //   QAvgPool / QMaxPool   Pool(Dequantize(x))                  -> Dequantize(Pool(x))
                //   QConcat        Concat(Dequantize(x_i) ...), equal scales   -> Dequantize(Concat(x_i ...))
                //   DQandQ         Quantize(Dequantize(x)), equal scales       -> x
                // The reference's last pattern (QuantizedDot -> QuantizedMatmul with a transposed
                // second operand, the layout its GEMM library wants) has no counterpart: this
                // backend repacks a constant second operand once at compile time.
                class NGRAPH_API HIPQuantFusion : public ngraph::pass::FunctionPass
                {
                public:
                    bool run_on_function(std::shared_ptr<Function> f) override;
                };
            }
        }
    }
}
