// ref_shim.cpp -- TEST INFRASTRUCTURE.  C entry points over the *real* nGraph reference kernels.
//
// Compiled only where the nGraph source tree is present (oracle/Makefile, target `ref`), straight
// from the reference's own headers and seven small .cpp files; the result goes to oracle/_ref/.
// It validates the C restatement in hipq_oracle.c and serves as the CPU baseline of the
// benchmark.  Signatures take flat arrays so that ctypes can call them.
#include <cstddef>
#include <cstdint>
#include <vector>

#include "ngraph/axis_set.hpp"
#include "ngraph/coordinate_diff.hpp"
#include "ngraph/runtime/reference/avg_pool.hpp"
#include "ngraph/runtime/reference/batch_mat_mul.hpp"
#include "ngraph/runtime/reference/convolution.hpp"
#include "ngraph/runtime/reference/dequantize.hpp"
#include "ngraph/runtime/reference/dot.hpp"
#include "ngraph/runtime/reference/max_pool.hpp"
#include "ngraph/runtime/reference/erf.hpp"
#include "ngraph/runtime/reference/quantize.hpp"
#include "ngraph/runtime/reference/softmax.hpp"
#include "ngraph/runtime/reference/sum.hpp"
#include "ngraph/shape.hpp"
#include "ngraph/strides.hpp"

using namespace ngraph;

namespace
{
    Shape make_shape(const int64_t* v, int n)
    {
        Shape s;
        for (int i = 0; i < n; ++i)
            s.push_back(static_cast<size_t>(v[i]));
        return s;
    }
    Strides make_strides(const int64_t* v, int n)
    {
        Strides s;
        for (int i = 0; i < n; ++i)
            s.push_back(static_cast<size_t>(v[i]));
        return s;
    }
    CoordinateDiff make_diff(const int64_t* v, int n)
    {
        CoordinateDiff s;
        for (int i = 0; i < n; ++i)
            s.push_back(static_cast<std::ptrdiff_t>(v[i]));
        return s;
    }
    AxisSet make_axes(uint32_t mask)
    {
        AxisSet a;
        for (size_t i = 0; i < 32; ++i)
            if (mask & (1u << i))
                a.insert(i);
        return a;
    }

    template <typename IN, typename FILT, typename OUT>
    void conv(const void* in,
              const void* filt,
              void* out,
              const Shape& is,
              const Shape& fs,
              const Shape& os,
              const Strides& st,
              const Strides& dl,
              const CoordinateDiff& pb,
              const CoordinateDiff& pa,
              const Strides& dd,
              const float* isc,
              const void* izp,
              const float* fsc,
              const void* fzp,
              const float* osc,
              const void* ozp)
    {
        runtime::reference::convolution<IN, FILT, OUT, int32_t>(static_cast<const IN*>(in),
                                                                static_cast<const FILT*>(filt),
                                                                static_cast<OUT*>(out),
                                                                is,
                                                                fs,
                                                                os,
                                                                st,
                                                                dl,
                                                                pb,
                                                                pa,
                                                                dd,
                                                                isc,
                                                                static_cast<const IN*>(izp),
                                                                fsc,
                                                                static_cast<const FILT*>(fzp),
                                                                osc,
                                                                static_cast<const OUT*>(ozp));
    }

    template <typename A, typename B, typename OUT>
    void dot(const void* a,
             const void* b,
             void* out,
             const Shape& as,
             const Shape& bs,
             const Shape& os,
             const float* asc,
             const void* azp,
             const float* bsc,
             const void* bzp,
             const float* osc,
             const void* ozp)
    {
        runtime::reference::dot<A, B, OUT, int32_t>(static_cast<const A*>(a),
                                                    static_cast<const B*>(b),
                                                    static_cast<OUT*>(out),
                                                    as,
                                                    bs,
                                                    os,
                                                    1,
                                                    asc,
                                                    static_cast<const A*>(azp),
                                                    bsc,
                                                    static_cast<const B*>(bzp),
                                                    osc,
                                                    static_cast<const OUT*>(ozp));
    }
}

// dtype codes: 0 u8, 1 i8, 2 i32, 3 f32, 4 f64 (same as include/hipq.h)
extern "C" {

// data [N,C,spatial...], filter [K,C,spatial...]; type combinations of
// src/ngraph/runtime/interpreter/int_executable.hpp:1461-1549.  Returns 0, or 2 if unsupported.
__attribute__((visibility("default"))) int ref_quantized_convolution(int n_spatial,
                                                                       const int64_t* data_shape,
                                                                       const int64_t* filter_shape,
                                                                       const int64_t* out_shape,
                                                                       const int64_t* stride,
                                                                       const int64_t* dilation,
                                                                       const int64_t* pad_below,
                                                                       const int64_t* pad_above,
                                                                       const int64_t* data_dilation,
                                                                       int data_t,
                                                                       int filter_t,
                                                                       int out_t,
                                                                       const void* data,
                                                                       const void* filter,
                                                                       const float* data_scale,
                                                                       const void* data_zp,
                                                                       const float* filter_scale,
                                                                       const void* filter_zp,
                                                                       const float* out_scale,
                                                                       const void* out_zp,
                                                                       void* out)
{
    Shape is = make_shape(data_shape, n_spatial + 2);
    Shape fs = make_shape(filter_shape, n_spatial + 2);
    Shape os = make_shape(out_shape, n_spatial + 2);
    Strides st = make_strides(stride, n_spatial);
    Strides dl = make_strides(dilation, n_spatial);
    Strides dd = make_strides(data_dilation, n_spatial);
    CoordinateDiff pb = make_diff(pad_below, n_spatial);
    CoordinateDiff pa = make_diff(pad_above, n_spatial);
#define CONV_ARGS                                                                                  \
    data, filter, out, is, fs, os, st, dl, pb, pa, dd, data_scale, data_zp, filter_scale,         \
        filter_zp, out_scale, out_zp
    if (data_t == 0 && filter_t == 1 && out_t == 1)
        conv<uint8_t, int8_t, int8_t>(CONV_ARGS);
    else if (data_t == 0 && filter_t == 0 && out_t == 0)
        conv<uint8_t, uint8_t, uint8_t>(CONV_ARGS);
    else if (data_t == 0 && filter_t == 1 && out_t == 2)
        conv<uint8_t, int8_t, int32_t>(CONV_ARGS);
    else if (data_t == 0 && filter_t == 0 && out_t == 2)
        conv<uint8_t, uint8_t, int32_t>(CONV_ARGS);
    else
        return 2;
#undef CONV_ARGS
    return 0;
}

// a [M,K], b [K,N]; combinations of int_executable.hpp:1573-1645
__attribute__((visibility("default"))) int ref_quantized_dot(int64_t M,
                                                               int64_t K,
                                                               int64_t N,
                                                               int a_t,
                                                               int b_t,
                                                               int out_t,
                                                               const void* a,
                                                               const void* b,
                                                               const float* a_scale,
                                                               const void* a_zp,
                                                               const float* b_scale,
                                                               const void* b_zp,
                                                               const float* out_scale,
                                                               const void* out_zp,
                                                               void* out)
{
    Shape as{static_cast<size_t>(M), static_cast<size_t>(K)};
    Shape bs{static_cast<size_t>(K), static_cast<size_t>(N)};
    Shape os{static_cast<size_t>(M), static_cast<size_t>(N)};
#define DOT_ARGS a, b, out, as, bs, os, a_scale, a_zp, b_scale, b_zp, out_scale, out_zp
    if (a_t == 0 && b_t == 1 && out_t == 1)
        dot<uint8_t, int8_t, int8_t>(DOT_ARGS);
    else if (a_t == 0 && b_t == 0 && out_t == 0)
        dot<uint8_t, uint8_t, uint8_t>(DOT_ARGS);
    else if (a_t == 0 && b_t == 0 && out_t == 2)
        dot<uint8_t, uint8_t, int32_t>(DOT_ARGS);
    else if (a_t == 0 && b_t == 1 && out_t == 2)
        dot<uint8_t, int8_t, int32_t>(DOT_ARGS);
    else
        return 2;
#undef DOT_ARGS
    return 0;
}

__attribute__((visibility("default"))) int ref_quantize(int rank,
                                                          const int64_t* shape,
                                                          uint32_t axes_mask,
                                                          int real_t,
                                                          int quant_t,
                                                          int round_mode,
                                                          const void* in,
                                                          const void* scale,
                                                          const void* zp,
                                                          void* out)
{
    Shape s = make_shape(shape, rank);
    AxisSet axes = make_axes(axes_mask);
    Shape ss;
    for (int i = 0; i < rank; ++i)
        if (axes_mask & (1u << i))
            ss.push_back(s[i]);
    auto mode = static_cast<op::v0::Quantize::RoundMode>(round_mode);
#define Q(REAL, QUANT)                                                                             \
    runtime::reference::quantize<REAL, QUANT>(static_cast<const REAL*>(in),                        \
                                              static_cast<const REAL*>(scale),                     \
                                              static_cast<const QUANT*>(zp),                       \
                                              static_cast<QUANT*>(out),                            \
                                              s,                                                   \
                                              ss,                                                  \
                                              axes,                                                \
                                              mode)
    if (real_t == 3 && quant_t == 0)
        Q(float, uint8_t);
    else if (real_t == 3 && quant_t == 1)
        Q(float, int8_t);
    else if (real_t == 3 && quant_t == 2)
        Q(float, int32_t);
    else if (real_t == 4 && quant_t == 0)
        Q(double, uint8_t);
    else if (real_t == 4 && quant_t == 1)
        Q(double, int8_t);
    else if (real_t == 4 && quant_t == 2)
        Q(double, int32_t);
    else
        return 2;
#undef Q
    return 0;
}

__attribute__((visibility("default"))) int ref_dequantize(int rank,
                                                            const int64_t* shape,
                                                            uint32_t axes_mask,
                                                            int real_t,
                                                            int quant_t,
                                                            const void* in,
                                                            const void* scale,
                                                            const void* zp,
                                                            void* out)
{
    Shape s = make_shape(shape, rank);
    AxisSet axes = make_axes(axes_mask);
    Shape ss;
    for (int i = 0; i < rank; ++i)
        if (axes_mask & (1u << i))
            ss.push_back(s[i]);
#define DQ(QUANT, REAL)                                                                            \
    runtime::reference::dequantize<QUANT, REAL>(static_cast<const QUANT*>(in),                     \
                                                static_cast<const REAL*>(scale),                   \
                                                static_cast<const QUANT*>(zp),                     \
                                                static_cast<REAL*>(out),                           \
                                                s,                                                 \
                                                ss,                                                \
                                                axes)
    if (real_t == 3 && quant_t == 0)
        DQ(uint8_t, float);
    else if (real_t == 3 && quant_t == 1)
        DQ(int8_t, float);
    else if (real_t == 3 && quant_t == 2)
        DQ(int32_t, float);
    else if (real_t == 4 && quant_t == 0)
        DQ(uint8_t, double);
    else if (real_t == 4 && quant_t == 1)
        DQ(int8_t, double);
    else if (real_t == 4 && quant_t == 2)
        DQ(int32_t, double);
    else
        return 2;
#undef DQ
    return 0;
}

// runtime::reference::max_pool<T> / avg_pool<T> on NCX tensors; dtype codes as in hipq.h; op 0 = max, 1 = avg
__attribute__((visibility("default"))) int ref_pool(int op,
                                                      int dtype,
                                                      int n_spatial,
                                                      const int64_t* arg_shape,
                                                      const int64_t* out_shape,
                                                      const int64_t* window,
                                                      const int64_t* stride,
                                                      const int64_t* pad_below,
                                                      const int64_t* pad_above,
                                                      int include_padding,
                                                      const void* in,
                                                      void* out)
{
    Shape as = make_shape(arg_shape, n_spatial + 2), os = make_shape(out_shape, n_spatial + 2);
    Shape w = make_shape(window, n_spatial), pb = make_shape(pad_below, n_spatial), pa = make_shape(pad_above, n_spatial);
    Strides st;
    for (int i = 0; i < n_spatial; ++i)
        st.push_back(static_cast<size_t>(stride[i]));
    try
    {
#define P(T)                                                                                       \
    if (op == 0)                                                                                   \
        runtime::reference::max_pool<T>(static_cast<const T*>(in), static_cast<T*>(out), as, os, w, st, pb, pa); \
    else                                                                                           \
        runtime::reference::avg_pool<T>(static_cast<const T*>(in), static_cast<T*>(out), as, os, w, st, pb, pa, include_padding != 0)
        switch (dtype)
        {
        case 0: P(uint8_t); break;
        case 1: P(int8_t); break;
        case 2: P(int32_t); break;
        case 3: P(float); break;
        default: return -1;
        }
#undef P
    }
    catch (const std::exception&)
    {
        return -2;
    }
    return 0;
}

// runtime::reference::softmax<float> over the axes whose bit is set in axes_mask
__attribute__((visibility("default"))) int ref_softmax_f32(const float* in, float* out, const int64_t* shape, int rank, uint32_t axes_mask)
{
    Shape sh = make_shape(shape, rank);
    AxisSet axes;
    for (int i = 0; i < rank; ++i)
        if (axes_mask & (1u << i))
            axes.insert(static_cast<size_t>(i));
    try
    {
        runtime::reference::softmax<float>(in, out, sh, axes);
    }
    catch (const std::exception&)
    {
        return -2;
    }
    return 0;
}

// runtime::reference::sum<float> (the Kahan-compensated sequential sum LayerNorm's mean and variance use)
__attribute__((visibility("default"))) int ref_sum_f32(const float* in, float* out, const int64_t* shape, int rank, uint32_t axes_mask)
{
    Shape sh = make_shape(shape, rank);
    AxisSet axes;
    for (int i = 0; i < rank; ++i)
        if (axes_mask & (1u << i))
            axes.insert(static_cast<size_t>(i));
    try
    {
        runtime::reference::sum<float>(in, out, sh, axes);
    }
    catch (const std::exception&)
    {
        return -2;
    }
    return 0;
}

__attribute__((visibility("default"))) int ref_erf_f32(const float* in, float* out, int64_t count)
{
    runtime::reference::erf<float>(in, out, static_cast<size_t>(count));
    return 0;
}

// runtime::reference::batch_mat_mul<float>: a [batch, M, K], b [batch, K, N]
__attribute__((visibility("default"))) int ref_batch_mat_mul_f32(const float* a, const float* b, float* out, int64_t batch, int64_t M, int64_t K, int64_t N)
{
    try
    {
        runtime::reference::batch_mat_mul<float>(a,
                                                 b,
                                                 out,
                                                 Shape{static_cast<size_t>(batch), static_cast<size_t>(M), static_cast<size_t>(K)},
                                                 Shape{static_cast<size_t>(batch), static_cast<size_t>(K), static_cast<size_t>(N)},
                                                 Shape{static_cast<size_t>(batch), static_cast<size_t>(M), static_cast<size_t>(N)});
    }
    catch (const std::exception&)
    {
        return -2;
    }
    return 0;
}
}
