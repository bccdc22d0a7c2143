// Implicit-GEMM convolution on the i8 matrix cores: eligibility and launch (kernel in hipq_igemm.h).
#include "hipq_igemm.h"

namespace hipq
{
    bool conv_mfma_eligible(const ConvGeom& g)
    {
        if (g.in[0] != 1 || g.f[0] != 1 || g.out[0] != 1) // 1-D / 2-D only
            return false;
        if (g.dd[0] != 1 || g.dd[1] != 1 || g.dd[2] != 1)
            return false;
        if (g.filter_t != HIPQ_I8 || (g.data_t != HIPQ_U8 && g.data_t != HIPQ_I8))
            return false;
        if (g.C % 16 != 0)
            return false;
        if (!fits_i32(g.in_count()) || !fits_i32(g.out_count()) || !fits_i32(g.K * g.C * g.taps()))
            return false;
        if (g.K > 65535 * 64)
            return false;
        if (g.out_t != HIPQ_U8 && g.out_t != HIPQ_I8 && g.out_t != HIPQ_I32)
            return false;
        // the kernel keeps window origins in 16 bits
        for (int i = 1; i < 3; ++i)
            if (g.out[i] * g.st[i] + (g.pb[i] < 0 ? -g.pb[i] : g.pb[i]) + g.f[i] * g.dl[i] >= 32000 || g.in[i] >= 32000)
                return false;
        return true;
    }

    int launch_conv_mfma(const ConvGeom& g,
                         const void* data_nxc,
                         const void* packed,
                         const ZeroPoints& zp,
                         const Epilogue& epi,
                         void* out,
                         bool out_ncx,
                         hipStream_t s)
    {
        HIPQ_REQUIRE(conv_mfma_eligible(g), "shape not eligible for the MFMA convolution");
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(data_nxc) & 15) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(out) & 15) == 0,
                     "MFMA convolution needs 16-byte aligned tensors");
        ConvX xl;
        xl.x = static_cast<const uint8_t*>(data_nxc);
        xl.H = static_cast<int32_t>(g.in[1]);
        xl.W = static_cast<int32_t>(g.in[2]);
        xl.C = static_cast<int32_t>(g.C);
        xl.Q = static_cast<int32_t>(g.out[2]);
        xl.R = static_cast<int32_t>(g.f[1]);
        xl.S = static_cast<int32_t>(g.f[2]);
        xl.sh = static_cast<int32_t>(g.st[1]);
        xl.sw = static_cast<int32_t>(g.st[2]);
        xl.dh = static_cast<int32_t>(g.dl[1]);
        xl.dw = static_cast<int32_t>(g.dl[2]);
        xl.pbh = static_cast<int32_t>(g.pb[1]);
        xl.pbw = static_cast<int32_t>(g.pb[2]);
        xl.PQ = g.out[1] * g.out[2];
        xl.bytes = static_cast<uint32_t>(g.in_count());
        const int64_t M = g.N * xl.PQ;
        xl.by_pq = fast_div(xl.PQ);
        if (M >= (1ll << 31))
            xl.by_pq.sh = 0xffffffffu;
        xl.by_q = fast_div(xl.Q);
        xl.by_c = fast_div(xl.C);
        xl.by_s = fast_div(xl.S);
        const int32_t N = static_cast<int32_t>(g.K);
        const int32_t Kred = static_cast<int32_t>(g.C * g.taps());
        const int8_t* w = static_cast<const int8_t*>(packed);
        const int32_t* wsum =
            reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(packed) + align_up(static_cast<size_t>(g.K) * Kred, 256));
        OutMap om{out_ncx ? 1 : 0, N, xl.PQ};
        const int xu = g.data_t == HIPQ_U8 ? 1 : 0;
        // a 1 x 1 filter over every pixel: the channels-last data is the [pixels][C] matrix itself
        if (!out_ncx && g.taps() == 1 && g.st[1] == 1 && g.st[2] == 1 && g.pb[1] == 0 && g.pb[2] == 0 && g.out[1] == g.in[1] && g.out[2] == g.in[2] &&
            g.C % 16 == 0)
            return launch_rows_mfma(data_nxc, xu != 0, w, wsum, M, N, Kred, zp, epi, out, s, "conv_mfma_i8_32x32x32");
        // Channel counts in whole 64-byte slices take the kernels that load straight into LDS (on
        // ResNet-50's 3 x 3 and strided layers about 8 % faster than the register-staged ones);
        // HIPQ_NO_CONV_DMA=1 keeps windows on the register-staged kernels.
        if (!out_ncx && g.C % 64 == 0 && M < (1ll << 31) && getenv("HIPQ_NO_CONV_DMA") == nullptr)
        {
            ConvU xc;
            xc.cx = xl;
            xc.x = xl.x;
            xc.bytes = xl.bytes;
            const int rc = launch_uniform(xc, w, wsum, M, N, Kred, xu, zp, epi, om, out, s, "conv_mfma_i8_32x32x32");
            if (rc != HIPQ_ERR_UNSUPPORTED)
                return rc;
        }
        if (out_ncx)
            return launch_epilogue<ConvX, true>(xl, w, wsum, M, N, Kred, xu, zp, epi, om, out, s, "conv_mfma_i8_32x32x32");
        return launch_epilogue<ConvX, false>(xl, w, wsum, M, N, Kred, xu, zp, epi, om, out, s, "conv_mfma_i8_32x32x32");
    }
}
