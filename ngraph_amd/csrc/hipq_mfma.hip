// int8 GEMM and implicit-GEMM convolution on the CDNA4 i8 matrix cores (v_mfma_i32_32x32x32_i8).
//
// out[m][n] = epilogue( sum_k (x[m][k] - x_zp) * w[n][k] )
//   x : the activation operand.  GEMM: a row-major [M][K] matrix.  Convolution: gathered on the
//       fly from channels-last data, m = (image, out_y, out_x), k = (filter_y, filter_x, channel).
//   w : the weights as [N][K] int8, K contiguous (for convolution: K,spatial,C order).
//
// The matrix cores multiply signed by signed bytes only, so unsigned activations are biased:
// x' = x ^ 0x80 = x - 128, and since  sum (x - zp) w = sum x' w + (128 - zp) * sum w  the
// kernel adds (128 - zp) * wsum[n] to each accumulator.  Padding taps are materialised as the
// byte `zp` (a real element equal to the zero point), which contributes (zp - zp) * w = 0 exactly
// as the reference's skipped tap does.
//
// Work split: a workgroup of 4 wavefronts computes a 128 (m) x 128 (n) tile, each wavefront a
// 64 x 64 quadrant as 2 x 2 MFMA tiles.  Operands are staged through LDS in 64-byte K slices,
// double buffered: global loads of slice i+1 are in flight while slice i feeds the MFMAs.
// LDS rows are 64 bytes with the 16-byte chunk index XOR-swizzled by (row >> 1) & 3, which makes
// both the 16-byte stores and the 16-byte fragment reads free of bank conflicts.
//
// The weights feed MFMA source A (rows) and the activations source B (columns), so that a lane's
// four consecutive accumulator registers are four consecutive output channels of one pixel: they
// pack into one 4-byte store in a channels-last / row-major output.
#include "hipq_common.h"

namespace hipq
{
    typedef int v4i __attribute__((ext_vector_type(4)));
    typedef int v16i __attribute__((ext_vector_type(16)));

    constexpr int BM = 128; // activation rows per workgroup
    constexpr int BN = 128; // weight rows (output channels) per workgroup
    constexpr int BK = 64;  // reduction bytes per LDS slice

    __device__ __forceinline__ int lds_offset(int row, int chunk)
    {
        return row * BK + ((chunk ^ ((row >> 1) & 3)) << 4);
    }

    // ---- activation loaders ---------------------------------------------------------------------
    struct GemmX
    {
        const uint8_t* x;
        int32_t K;

        struct Row
        {
            const uint8_t* p;
            bool valid;
        };
        struct Cursor
        {
            int32_t kbyte;
        };
        __device__ void init_row(Row& r, int64_t m, int64_t M) const
        {
            r.valid = m < M;
            r.p = x + (r.valid ? m : 0) * static_cast<int64_t>(K);
        }
        __device__ void init_cursor(Cursor& c, int kbyte) const { c.kbyte = kbyte; }
        __device__ void advance(Cursor& c, int bytes) const { c.kbyte += bytes; }
        __device__ v4i load(const Row& r, const Cursor& c, int fill) const
        {
            if (!r.valid || c.kbyte >= K)
                return v4i{fill, fill, fill, fill};
            return *reinterpret_cast<const v4i*>(r.p + c.kbyte);
        }
        // slow path: exact accumulator of one output, any zero points
        __device__ int32_t direct(int64_t m, const int8_t* wrow, int32_t xzp, int32_t wzp, bool x_unsigned) const
        {
            const uint8_t* p = x + m * static_cast<int64_t>(K);
            int32_t acc = 0;
            for (int32_t k = 0; k < K; ++k)
            {
                int32_t a = x_unsigned ? static_cast<int32_t>(p[k]) : static_cast<int32_t>(static_cast<int8_t>(p[k]));
                acc += (a - xzp) * (static_cast<int32_t>(wrow[k]) - wzp);
            }
            return acc;
        }
    };

    struct ConvX
    {
        const uint8_t* x; // [N][H][W][C]
        int32_t H, W, C, Q, R, S, sh, sw, dh, dw, pbh, pbw;
        int64_t PQ;

        struct Row
        {
            int32_t base; // byte offset of the image
            int32_t iy0, ix0;
            bool valid;
        };
        struct Cursor
        {
            int32_t r, s, c;
        };
        __device__ void init_row(Row& rw, int64_t m, int64_t M) const
        {
            rw.valid = m < M;
            int64_t mm = rw.valid ? m : 0;
            int64_t n = mm / PQ;
            int32_t rem = static_cast<int32_t>(mm - n * PQ);
            int32_t p = rem / Q;
            int32_t q = rem - p * Q;
            rw.base = static_cast<int32_t>(n) * H * W * C;
            rw.iy0 = p * sh - pbh;
            rw.ix0 = q * sw - pbw;
        }
        __device__ void init_cursor(Cursor& c, int kbyte) const
        {
            int tap = kbyte / C;
            c.c = kbyte - tap * C;
            c.r = tap / S;
            c.s = tap - c.r * S;
        }
        __device__ void advance(Cursor& c, int bytes) const
        {
            c.c += bytes;
            while (c.c >= C)
            {
                c.c -= C;
                if (++c.s == S)
                {
                    c.s = 0;
                    ++c.r;
                }
            }
        }
        __device__ v4i load(const Row& rw, const Cursor& c, int fill) const
        {
            int32_t y = rw.iy0 + c.r * dh;
            int32_t xx = rw.ix0 + c.s * dw;
            if (!rw.valid || c.r >= R || static_cast<uint32_t>(y) >= static_cast<uint32_t>(H) ||
                static_cast<uint32_t>(xx) >= static_cast<uint32_t>(W))
                return v4i{fill, fill, fill, fill};
            return *reinterpret_cast<const v4i*>(x + rw.base + (y * W + xx) * C + c.c);
        }
        __device__ int32_t direct(int64_t m, const int8_t* wrow, int32_t xzp, int32_t wzp, bool x_unsigned) const
        {
            Row rw;
            init_row(rw, m, m + 1);
            int32_t acc = 0;
            for (int32_t r = 0; r < R; ++r)
                for (int32_t s = 0; s < S; ++s)
                {
                    int32_t y = rw.iy0 + r * dh, xx = rw.ix0 + s * dw;
                    if (static_cast<uint32_t>(y) >= static_cast<uint32_t>(H) || static_cast<uint32_t>(xx) >= static_cast<uint32_t>(W))
                        continue;
                    const uint8_t* p = x + rw.base + (y * W + xx) * C;
                    const int8_t* wp = wrow + (r * S + s) * C;
                    for (int32_t c = 0; c < C; ++c)
                    {
                        int32_t a = x_unsigned ? static_cast<int32_t>(p[c]) : static_cast<int32_t>(static_cast<int8_t>(p[c]));
                        acc += (a - xzp) * (static_cast<int32_t>(wp[c]) - wzp);
                    }
                }
            return acc;
        }
    };

    // Exact but slow tile for a non-zero weight zero point (w - wzp does not fit a signed byte).
    template <class XL>
    __device__ __noinline__ void slow_tile(const XL& xl,
                                           const int8_t* __restrict__ w,
                                           int64_t M,
                                           int32_t N,
                                           int32_t Kred,
                                           int32_t x_unsigned,
                                           int32_t xzp,
                                           int32_t wzp,
                                           const Epilogue& epi,
                                           void* __restrict__ out,
                                           int64_t m0,
                                           int32_t n0)
    {
        const EpiRegs er = epi_load(epi);
        for (int i = threadIdx.x; i < BM * BN; i += 256)
        {
            const int64_t m = m0 + i / BN;
            const int32_t n = n0 + i % BN;
            if (m < M && n < N)
            {
                int32_t a = xl.direct(m, w + static_cast<int64_t>(n) * Kred, xzp, wzp, x_unsigned != 0);
                store_out(out, epi.out_t, m * N + n, epi_apply(epi, er, a, n, m * N + n));
            }
        }
    }

    template <class XL>
    __global__ __launch_bounds__(256) void igemm_i8_kernel(XL xl,
                                                           const int8_t* __restrict__ w,
                                                           const int32_t* __restrict__ wsum,
                                                           int64_t M,
                                                           int32_t N,
                                                           int32_t Kred,
                                                           int32_t x_unsigned,
                                                           ZeroPoints zp,
                                                           Epilogue epi,
                                                           void* __restrict__ out)
    {
        __shared__ __attribute__((aligned(16))) uint8_t lds[2][2][BM * BK]; // [buffer][x / w][tile]

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int wn = wave & 1;
        const int wm = wave >> 1;
        const int64_t m0 = static_cast<int64_t>(blockIdx.x) * BM;
        const int32_t n0 = static_cast<int32_t>(blockIdx.y) * BN;

        const int32_t xzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t wzp = load_zp(zp.filter_zp, zp.filter_t);
        if (wzp != 0) // uniform across the grid
        {
            slow_tile(xl, w, M, N, Kred, x_unsigned, xzp, wzp, epi, out, m0, n0);
            return;
        }

        v16i acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[i][j][r] = 0;

        {
            const int lrow = tid >> 2;
            const int lchunk = tid & 3;
            const int xor_mask = x_unsigned ? static_cast<int>(0x80808080u) : 0;
            const int fill = (xzp & 0xFF) * 0x01010101;

            typename XL::Row xr[2];
            typename XL::Cursor cur;
            xl.init_row(xr[0], m0 + lrow, M);
            xl.init_row(xr[1], m0 + lrow + 64, M);
            xl.init_cursor(cur, lchunk * 16);
            const int8_t* wp[2];
            bool wv[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
            {
                int32_t n = n0 + lrow + 64 * i;
                wv[i] = n < N;
                wp[i] = w + static_cast<int64_t>(wv[i] ? n : 0) * Kred;
            }
            int32_t kb = lchunk * 16;

            v4i xreg[2], wreg[2];
            auto gload = [&]() {
#pragma unroll
                for (int i = 0; i < 2; ++i)
                {
                    v4i v = xl.load(xr[i], cur, fill);
                    xreg[i] = v4i{v[0] ^ xor_mask, v[1] ^ xor_mask, v[2] ^ xor_mask, v[3] ^ xor_mask};
                    wreg[i] = (wv[i] && kb < Kred) ? *reinterpret_cast<const v4i*>(wp[i] + kb) : v4i{0, 0, 0, 0};
                }
            };
            auto lstore = [&](int buf) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
                {
                    int off = lds_offset(lrow + 64 * i, lchunk);
                    *reinterpret_cast<v4i*>(&lds[buf][0][off]) = xreg[i];
                    *reinterpret_cast<v4i*>(&lds[buf][1][off]) = wreg[i];
                }
            };

            const int KT = (Kred + BK - 1) / BK;
            gload();
            lstore(0);
            __syncthreads();
            for (int kt = 0; kt < KT; ++kt)
            {
                const int buf = kt & 1;
                const bool more = kt + 1 < KT;
                if (more)
                {
                    xl.advance(cur, BK);
                    kb += BK;
                    gload();
                }
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
                {
                    v4i wf[2], xf[2];
                    const int chunk = ks * 2 + (lane >> 5);
#pragma unroll
                    for (int i = 0; i < 2; ++i)
                    {
                        wf[i] = *reinterpret_cast<const v4i*>(&lds[buf][1][lds_offset(wn * 64 + i * 32 + (lane & 31), chunk)]);
                        xf[i] = *reinterpret_cast<const v4i*>(&lds[buf][0][lds_offset(wm * 64 + i * 32 + (lane & 31), chunk)]);
                    }
#pragma unroll
                    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                        for (int mi = 0; mi < 2; ++mi)
                            acc[ni][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[ni], xf[mi], acc[ni][mi], 0, 0, 0);
                }
                if (more)
                    lstore(buf ^ 1);
                __syncthreads();
            }
        }

        // ---- epilogue: lane holds column m = lane % 32, rows n = 8*(r/4) + 4*(lane/32) + r%4 ----
        const EpiRegs er = epi_load(epi);
        const int32_t mult = (x_unsigned ? 128 : 0) - xzp;
        const bool out8 = (epi.out_t == HIPQ_U8 || epi.out_t == HIPQ_I8);
        const bool vec_ok = (N & 3) == 0;
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
        {
            const int64_t m = m0 + wm * 64 + mi * 32 + (lane & 31);
            if (m >= M)
                continue;
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
            {
#pragma unroll
                for (int g = 0; g < 4; ++g)
                {
                    const int32_t nb = n0 + wn * 64 + ni * 32 + 8 * g + 4 * (lane >> 5);
                    if (nb >= N)
                        continue;
                    int32_t v[4] = {0, 0, 0, 0};
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                    {
                        const int32_t n = nb + e;
                        if (n < N)
                        {
                            const int32_t a = acc[ni][mi][4 * g + e] + mult * wsum[n];
                            v[e] = epi_apply(epi, er, a, n, m * N + n);
                        }
                    }
                    const int64_t o = m * N + nb;
                    if (vec_ok) // nb is a multiple of 4, so nb + 3 < N and the store is aligned
                    {
                        if (out8)
                        {
                            uint32_t pk = (v[0] & 0xFF) | ((v[1] & 0xFF) << 8) | ((v[2] & 0xFF) << 16) |
                                          (static_cast<uint32_t>(v[3]) << 24);
                            *reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(out) + o) = pk;
                        }
                        else
                            *reinterpret_cast<v4i*>(static_cast<int32_t*>(out) + o) = v4i{v[0], v[1], v[2], v[3]};
                    }
                    else
                    {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (nb + e < N)
                                store_out(out, epi.out_t, o + e, v[e]);
                    }
                }
            }
        }
    }

    static bool fits_i32(int64_t v) { return v >= 0 && v < (1ll << 31); }

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
        if (g.K > 65535 * BN)
            return false;
        return true;
    }

    int launch_conv_mfma(const ConvGeom& g,
                         const void* data_nxc,
                         const void* packed,
                         const ZeroPoints& zp,
                         const Epilogue& epi,
                         void* out_nxc,
                         hipStream_t s)
    {
        HIPQ_REQUIRE(conv_mfma_eligible(g), "shape not eligible for the MFMA convolution");
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(data_nxc) & 15) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(out_nxc) & 15) == 0,
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
        const int64_t M = g.N * xl.PQ;
        const int32_t N = static_cast<int32_t>(g.K);
        const int32_t Kred = static_cast<int32_t>(g.C * g.taps());
        const int8_t* w = static_cast<const int8_t*>(packed);
        const int32_t* wsum =
            reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(packed) + align_up(static_cast<size_t>(g.K) * Kred, 256));
        dim3 grid(static_cast<unsigned>((M + BM - 1) / BM), static_cast<unsigned>((N + BN - 1) / BN));
        igemm_i8_kernel<ConvX><<<grid, 256, 0, s>>>(xl, w, wsum, M, N, Kred, g.data_t == HIPQ_U8 ? 1 : 0, zp, epi, out_nxc);
        return check_launch("conv_mfma_i8_32x32x32");
    }

    bool dot_mfma_eligible(const hipq_dot_desc_t& d)
    {
        if (d.b_t != HIPQ_I8 || (d.a_t != HIPQ_U8 && d.a_t != HIPQ_I8))
            return false;
        if (d.K % 16 != 0 || d.K <= 0 || d.M <= 0 || d.N <= 0)
            return false;
        if (!fits_i32(d.K) || !fits_i32(d.N) || d.N > 65535ll * BN)
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
        dim3 grid(static_cast<unsigned>((d.M + BM - 1) / BM), static_cast<unsigned>((d.N + BN - 1) / BN));
        igemm_i8_kernel<GemmX><<<grid, 256, 0, s>>>(xl,
                                                    static_cast<const int8_t*>(w_nk),
                                                    wsum,
                                                    d.M,
                                                    static_cast<int32_t>(d.N),
                                                    static_cast<int32_t>(d.K),
                                                    d.a_t == HIPQ_U8 ? 1 : 0,
                                                    zp,
                                                    epi,
                                                    out);
        return check_launch("dot_mfma_i8_32x32x32");
    }
}
