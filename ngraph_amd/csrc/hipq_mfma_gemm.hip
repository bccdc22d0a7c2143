// int8 GEMM on the i8 matrix cores: eligibility and launch (kernel in hipq_igemm.h).
#include "hipq_igemm.h"

namespace hipq
{
    bool dot_mfma_eligible(const hipq_dot_desc_t& d)
    {
        if (d.b_t != HIPQ_I8 || (d.a_t != HIPQ_U8 && d.a_t != HIPQ_I8))
            return false;
        if (d.K % 16 != 0 || d.K <= 0 || d.M <= 0 || d.N <= 0)
            return false;
        if (!fits_i32(d.K) || !fits_i32(d.N) || d.N > 65535ll * 64 || !fits_i32(d.M * d.K) || !fits_i32(d.N * d.K))
            return false;
        return true;
    }

    int launch_dot_mfma(const hipq_dot_desc_t& d,
                        const void* a,
                        const void* w_nk,
                        const int32_t* wsum,
                        const ZeroPoints& zp,
                        const Epilogue& epi,
                        void* out,
                        hipStream_t s)
    {
        HIPQ_REQUIRE(dot_mfma_eligible(d), "shape not eligible for the MFMA dot");
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w_nk) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(out) & 15) == 0,
                     "MFMA dot needs 16-byte aligned tensors");
        GemmX xl;
        xl.x = static_cast<const uint8_t*>(a);
        xl.K = static_cast<int32_t>(d.K);
        xl.bytes = static_cast<uint32_t>(d.M * d.K);
        OutMap om{0, static_cast<int32_t>(d.N), 1};
        return launch_epilogue<GemmX, false>(xl, static_cast<const int8_t*>(w_nk), wsum, d.M, static_cast<int32_t>(d.N),
                                         static_cast<int32_t>(d.K), d.a_t == HIPQ_U8 ? 1 : 0, zp, epi, om, out, s, "dot_mfma_i8_32x32x32");
    }
}
