// Quantize arithmetic of one element, shared by the Quantize kernels and by the kernels that
// quantize what they have just computed (LayerNorm, Gelu with a quantized output).
// Follows src/ngraph/runtime/reference/quantize.hpp:29-117 of the nGraph tree: true IEEE division
// by the scale, the reference's floor/ceil rounding formulas, zero point added in REAL, clamp in
// REAL, then the cast.
#pragma once
#include "hipq_common.h"

namespace hipq
{
    // ---- rounding (quantize.hpp:51-103), literal ----------------------------------------------
    template <typename REAL>
    __device__ __forceinline__ REAL round_by_mode(REAL q, int mode)
    {
        const REAL half = static_cast<REAL>(0.5);
        const REAL zero = static_cast<REAL>(0.0);
        switch (mode)
        {
        case HIPQ_ROUND_NEAREST_TOWARD_INFINITY:
        {
            REAL a = floor(fabs(q) + half);
            return (q < zero) ? -a : a;
        }
        case HIPQ_ROUND_NEAREST_TOWARD_ZERO:
        {
            REAL a = ceil(fabs(q) - half);
            return (q < zero) ? -a : a;
        }
        case HIPQ_ROUND_NEAREST_UPWARD: return floor(q + half);
        case HIPQ_ROUND_NEAREST_DOWNWARD: return ceil(q - half);
        case HIPQ_ROUND_NEAREST_TOWARD_EVEN:
        {
            REAL up = floor(q + half);
            REAL dn = ceil(q - half);
            // fmod(up, 2.0) == 0.0  <=>  up/2 is an integer (exact: halving never rounds here)
            REAL h = up * half;
            return (floor(h) == h) ? up : dn;
        }
        case HIPQ_ROUND_TOWARD_INFINITY:
        {
            REAL a = ceil(fabs(q));
            return (q < zero) ? -a : a;
        }
        case HIPQ_ROUND_TOWARD_ZERO:
        {
            REAL a = floor(fabs(q));
            return (q < zero) ? -a : a;
        }
        case HIPQ_ROUND_UP: return ceil(q);
        case HIPQ_ROUND_DOWN: return floor(q);
        default: return q;
        }
    }

    template <typename QUANT>
    struct QLimits;
    template <>
    struct QLimits<uint8_t>
    {
        static constexpr double lo = 0.0, hi = 255.0;
    };
    template <>
    struct QLimits<int8_t>
    {
        static constexpr double lo = -128.0, hi = 127.0;
    };
    template <>
    struct QLimits<int32_t>
    {
        static constexpr double lo = -2147483648.0, hi = 2147483647.0;
    };

    __device__ __forceinline__ float ieee_div(float a, float b) { return __fdiv_rn(a, b); }
    __device__ __forceinline__ double ieee_div(double a, double b) { return __ddiv_rn(a, b); }

    __device__ __forceinline__ int32_t cast_x86(float q) { return cvtt_x86(q); }
    __device__ __forceinline__ int32_t cast_x86(double q)
    {
        if (!(q < 2147483648.0) || q <= -2147483649.0)
            return INT32_MIN;
        return static_cast<int32_t>(q);
    }

    template <typename REAL, typename QUANT>
    __device__ __forceinline__ QUANT quantize_one(REAL x, REAL s, QUANT zp, int mode)
    {
        REAL q = ieee_div(x, s);                                   // quantize.hpp:47-48
        q = round_by_mode<REAL>(q, mode);                          // :51-103
        q = q + static_cast<REAL>(zp);                             // :106
        const REAL lo = static_cast<REAL>(QLimits<QUANT>::lo);     // :109-112
        const REAL hi = static_cast<REAL>(QLimits<QUANT>::hi);
        q = (q < lo) ? lo : q;
        q = (hi < q) ? hi : q;
        return static_cast<QUANT>(cast_x86(q));                    // :115
    }

}
