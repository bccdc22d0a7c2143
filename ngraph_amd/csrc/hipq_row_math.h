// Row reductions over groups of lanes and the Softmax arithmetic of one row piece, shared by the
// Softmax kernels and by the attention kernel that applies Softmax to scores it has just computed:
// both must round alike, sums included, so both call these.
#pragma once
#include <cmath>

#include "hipq_common.h"

namespace hipq
{
    typedef float row_f4 __attribute__((ext_vector_type(4)));

    // reductions over aligned groups of W lanes of a wavefront
    template <int W = 64>
    __device__ __forceinline__ float wave_max(float v)
    {
#pragma unroll
        for (int o = W / 2; o > 0; o >>= 1)
            v = fmaxf(v, __shfl_xor(v, o));
        return v;
    }
    template <int W = 64>
    __device__ __forceinline__ float wave_sum(float v)
    {
#pragma unroll
        for (int o = W / 2; o > 0; o >>= 1)
            v += __shfl_xor(v, o);
        return v;
    }

    // Softmax of a row of at most 4 W elements held one 16-byte piece a lane by W neighbouring lanes
    // (src/ngraph/runtime/reference/softmax.hpp:31-57): exp(x - max) / sum(exp(x - max)); with `scaled`
    // the input is Multiply(x, c), the product rounded to f32 as the Multiply op rounds it.  Lanes
    // past the row's end pass live = false.  The sum: a lane's four terms in order, then the lanes'
    // sums through the butterfly of wave_sum.
    template <int W>
    __device__ __forceinline__ row_f4 softmax_piece(row_f4 v, bool live, bool scaled, float c)
    {
        if (!live)
            v = row_f4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
        else if (scaled)
            v = row_f4{__fmul_rn(v[0], c), __fmul_rn(v[1], c), __fmul_rn(v[2], c), __fmul_rn(v[3], c)};
        const float m = wave_max<W>(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])));
        float s = 0.0f;
#pragma unroll
        for (int e = 0; e < 4; ++e)
        {
            v[e] = live ? expf(v[e] - m) : 0.0f;
            s += v[e];
        }
        s = wave_sum<W>(s);
        return row_f4{v[0] / s, v[1] / s, v[2] / s, v[3] / s};
    }
    // a / b rounded as the division rounds it, from r = fl(1 / b): q0 = a r, e = a - b q0 (exact in a fused
    // multiply-add), q = q0 + e r -- three instructions where the division sequence takes eleven.
    // (Markstein's correction: with a correctly rounded reciprocal the result is the correctly rounded
    // quotient as long as nothing overflows or goes subnormal; checked on the CPU against the division
    // for all 2^23 mantissas of a with b = float(sqrt(2)), and for 2 x 10^8 random pairs.)  Callers keep
    // infinities and zero divisors away from it.
    __device__ __forceinline__ float div_by_reciprocal(float a, float b, float r)
    {
        const float q0 = __fmul_rn(a, r);
        return fmaf(fmaf(-b, q0, a), r, q0);
    }

    // Gelu as the reference decomposes it (src/ngraph/op/gelu.cpp:46-60):
    // (0.5 * x) * (1 + erf(x / float(sqrt(2.0)))), every step rounded to f32.  Shared by the Gelu
    // kernel and by the GEMM epilogue that applies Gelu to what it has just computed.
    __device__ __forceinline__ float gelu1(float x)
    {
        const float sqrt_two = 1.41421354f; // float(std::sqrt(2.0))
        const float r = 0.70710677f;        // fl(1 / sqrt_two)
        // x / sqrt_two, bit for bit; an infinite x stays itself, and where the quotient would be
        // subnormal erf's argument is so small that 1 + erf is 1 either way
        const float t = __builtin_isinf(x) ? x : div_by_reciprocal(x, sqrt_two, r);
        return __fmul_rn(__fmul_rn(0.5f, x), __fadd_rn(1.0f, erff(t)));
    }

}
