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

    // ---- four elements at a time (the Quantize kernels, and the kernels that quantize what they have just computed)
    typedef float f32x4 __attribute__((ext_vector_type(4)));

    // ---- division with the reciprocal shared by the four elements of a group -------------------
    // The instruction sequence the compiler emits for an IEEE float division is
    //     r = rcp(s); r = fma(fma(-s, r, 1), r, r);
    //     q = x * r;  q = fma(fma(-s, q, x), r, q);  q = fma(fma(-s, q, x), r, q);
    // wrapped in v_div_scale / v_div_fmas / v_div_fixup, which rescale the operands when an
    // exponent is extreme and patch the special cases (zero, Inf, NaN, denormal).  For a divisor
    // with 2^-30 <= |s| <= 2^30 and a dividend with 2^-60 <= |x| < 2^30 neither does anything, so
    // the bare sequence returns the same bits, and the first line depends on s alone.  A dividend
    // below 2^-60 gives a quotient below 2^-30 in magnitude from either sequence: it rounds to
    // zero whichever bits it has.  Groups outside these ranges take the compiler's division.
    __device__ __forceinline__ bool shared_reciprocal_ok(f32x4 x, float s)
    {
        const float big = 1073741824.0f;       // 2^30
        const float small = 9.31322574615478515625e-10f; // 2^-30
        // the sum is NaN or Inf if any element is, and bounds every |x|
        float sum = (__builtin_fabsf(x[0]) + __builtin_fabsf(x[1])) + (__builtin_fabsf(x[2]) + __builtin_fabsf(x[3]));
        float a = __builtin_fabsf(s);
        return (sum < big) & (__builtin_amdgcn_fmed3f(a, small, big) == a);
    }

    // Four elements to four bytes, round-half-even, for a group that passed shared_reciprocal_ok.
    // v_cvt_pk_u8_f32 converts with saturation to 0..255 and places the byte, i.e. the clamp, the
    // cast and the packing in one instruction; signed outputs are computed 128 higher and flipped
    // back with one XOR (the sum rint(q) + z is exact wherever it lies near the clamp range).
    template <typename QUANT>
    __device__ __forceinline__ uint32_t quantize4_shared_reciprocal(f32x4 x, float s, float z)
    {
        const bool is_signed = QLimits<QUANT>::lo < 0.0;
        float zz = is_signed ? z + 128.0f : z;
        float r = __builtin_amdgcn_rcpf(s);
        float e = __builtin_fmaf(-s, r, 1.0f);
        r = __builtin_fmaf(e, r, r);
        uint32_t packed = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
            float q = __fmul_rn(x[k], r);
            float t = __builtin_fmaf(-s, q, x[k]);
            q = __builtin_fmaf(t, r, q);
            t = __builtin_fmaf(-s, q, x[k]);
            q = __builtin_fmaf(t, r, q);
            float v = __fadd_rn(__builtin_rintf(q), zz);
            packed = __builtin_amdgcn_cvt_pk_u8_f32(v, k, packed);
        }
        return is_signed ? packed ^ 0x80808080u : packed;
    }

    // For 8-bit outputs the reference's round-half-even formula equals rintf(): the two differ only
    // for |q| >= 2^23, where both lie beyond the clamp range whatever the zero point.
    template <typename QUANT, bool RNE>
    __device__ __forceinline__ uint32_t quantize4(f32x4 x, float s, float z, int mode)
    {
        if (RNE && shared_reciprocal_ok(x, s))
            return quantize4_shared_reciprocal<QUANT>(x, s, z);
        const float lo = static_cast<float>(QLimits<QUANT>::lo);
        const float hi = static_cast<float>(QLimits<QUANT>::hi);
        float q[4] = {x[0], x[1], x[2], x[3]};
        uint32_t packed = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e)
        {
            float v = __fdiv_rn(q[e], s);
            v = RNE ? rintf(v) : round_by_mode<float>(v, mode);
            v = __fadd_rn(v, z);
            v = (v < lo) ? lo : v;
            v = (hi < v) ? hi : v;
            int32_t iv = static_cast<int32_t>(v); // in range after the clamp (NaN aside)
            packed |= (static_cast<uint32_t>(iv) & 0xFFu) << (8 * e);
        }
        return packed;
    }

}
