// Convolutions over at most four input channels (a network's first layer) on the tile kernels that
// load straight into LDS: eligibility, the staged copy of the data, launch.
#include <cstdlib>

#include "hipq_igemm.h"

namespace hipq
{
    bool conv_rowpack_eligible(const ConvGeom& g, RowPack* rp)
    {
        if (g.in[0] != 1 || g.f[0] != 1 || g.out[0] != 1) // 1-D / 2-D only
            return false;
        for (int i = 0; i < 3; ++i)
            if (g.dd[i] != 1 || g.dl[i] != 1)
                return false;
        if (g.filter_t != HIPQ_I8 || (g.data_t != HIPQ_U8 && g.data_t != HIPQ_I8))
            return false;
        if (g.out_t != HIPQ_U8 && g.out_t != HIPQ_I8)
            return false;
        if (g.C < 1 || g.C > 4 || g.f[2] > 8 || g.K % 16 != 0)
            return false;
        if (g.out_layout != HIPQ_LAYOUT_NXC && g.K > 1)
            return false;
        if (g.pb[1] < 0 || g.pb[2] < 0 || g.out[1] < 1 || g.out[2] < 1)
            return false;
        RowPack r;
        r.Hp = (g.out[1] - 1) * g.st[1] + g.f[1];
        r.Wp = (g.out[2] - 1) * g.st[2] + 8;
        r.kp = static_cast<int64_t>(align_up(static_cast<size_t>(g.f[1] * 32), 64));
        if (!fits_i32(g.N * r.Hp * r.Wp * 4 + 64) || !fits_i32(g.in_count()) || !fits_i32(g.out_count()) || !fits_i32(g.K * r.kp))
            return false;
        if (getenv("HIPQ_NO_ROWPACK") != nullptr || getenv("HIPQ_NO_PIPE") != nullptr || getenv("HIPQ_NO_DMA") != nullptr)
            return false;
        if (rp)
            *rp = r;
        return true;
    }

    // [N][C][H][W] or [N][H][W][C] bytes -> [N][Hp][Wp][4]: staged pixel (y, x) is input pixel
    // (y - pad_h, x - pad_w) where that exists; everything else, and the channels beyond C, hold the
    // data zero point.  One staged pixel (one dword) a lane and kStageRows staged rows (image, y) a
    // block column, their loads all issued before the first store: a block that moves one row
    // lives for one memory round trip, and a compute unit holds too few of those to cover it.
    constexpr int kStageRows = 8;
    __global__ __launch_bounds__(256) void stage_rows_kernel(const uint8_t* __restrict__ in, uint32_t* __restrict__ out, uint32_t rows, int32_t Hp, int32_t Wp, int32_t H, int32_t W,
                                                             int32_t Cc, int32_t pbh, int32_t pbw, int32_t in_ncx, const void* zp, int32_t zp_t)
    {
        const int32_t xp = static_cast<int32_t>(blockIdx.y) * 256 + static_cast<int32_t>(threadIdx.x);
        if (xp >= Wp)
            return;
        const uint32_t fill = (static_cast<uint32_t>(load_zp(zp, zp_t)) & 0xffu) * 0x01010101u;
        const int32_t x = xp - pbw;
        const int64_t X = static_cast<int64_t>(H) * W;
        const int64_t step = in_ncx ? X : 1;
        uint32_t v[kStageRows];
#pragma unroll
        for (int i = 0; i < kStageRows; ++i)
        {
            const uint32_t row = blockIdx.x * kStageRows + i; // image * Hp + yp
            v[i] = fill;
            if (row >= rows)
                continue;
            const uint32_t n = row / static_cast<uint32_t>(Hp);
            const int32_t y = static_cast<int32_t>(row - n * static_cast<uint32_t>(Hp)) - pbh;
            if (static_cast<uint32_t>(y) < static_cast<uint32_t>(H) && static_cast<uint32_t>(x) < static_cast<uint32_t>(W))
            {
                const int64_t pix = static_cast<int64_t>(y) * W + x;
                const uint8_t* p = in_ncx ? in + static_cast<int64_t>(n) * Cc * X + pix : in + (static_cast<int64_t>(n) * X + pix) * Cc;
                for (int c = 0; c < Cc; ++c)
                {
                    const uint32_t b = p[c * step];
                    v[i] = (v[i] & ~(0xffu << (8 * c))) | (b << (8 * c));
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kStageRows; ++i)
        {
            const uint32_t row = blockIdx.x * kStageRows + i;
            if (row < rows)
                out[static_cast<int64_t>(row) * Wp + xp] = v[i];
        }
    }

    // The same copy for data whose rows are whole aligned dwords: a lane takes four consecutive
    // pixels of one row -- one dword from each channel plane of [N][C][H][W] data, the 4 C contiguous
    // bytes of [N][H][W][C] data, instead of single bytes -- and writes their four staged pixels as
    // one 16-byte piece; kQuadRows rows a lane, every load issued
    // before the first store.  Quad j of a staged row covers input pixels 4j .. 4j + 3, that is
    // staged pixels 4j + pad_w .. 4j + pad_w + 3; quads run from -ceil(pad_w / 4) so that the left
    // padding is written too (pixels outside the staged row are dropped, outside the image filled).
    constexpr int kQuadRows = 4;
    struct __attribute__((packed, aligned(4))) Quad
    {
        uint32_t px[4];
    };
    template <int CC, bool NCX>
    __global__ __launch_bounds__(256) void stage_rows_quads_kernel(const uint8_t* __restrict__ in, uint32_t* __restrict__ out, uint32_t rows, int32_t Hp, int32_t Wp, int32_t H, int32_t W,
                                                                   int32_t pbh, int32_t pbw, int32_t first_quad, int32_t quads, const void* zp, int32_t zp_t)
    {
        const int32_t q = static_cast<int32_t>(blockIdx.y) * 64 + static_cast<int32_t>(threadIdx.x & 63);
        if (q >= quads)
            return;
        const int32_t x = (q + first_quad) * 4; // first input pixel of the quad; W is a multiple of 4, so a quad is inside the row or outside
        const bool x_in = x >= 0 && x < W;
        const uint32_t fill = (static_cast<uint32_t>(load_zp(zp, zp_t)) & 0xffu) * 0x01010101u;
        const int64_t X = static_cast<int64_t>(H) * W;
        const uint32_t row0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * kQuadRows;
        uint32_t word[kQuadRows][CC]; // NCX: the four pixels' bytes of channel c; NXC: bytes 4 c .. 4 c + 3 of the four pixels' run
        bool live[kQuadRows];
#pragma unroll
        for (int i = 0; i < kQuadRows; ++i)
        {
            const uint32_t row = row0 + i; // image * Hp + yp
#pragma unroll
            for (int c = 0; c < CC; ++c)
                word[i][c] = fill;
            live[i] = false;
            if (row >= rows || !x_in)
                continue;
            const uint32_t n = row / static_cast<uint32_t>(Hp);
            const int32_t y = static_cast<int32_t>(row - n * static_cast<uint32_t>(Hp)) - pbh;
            if (static_cast<uint32_t>(y) >= static_cast<uint32_t>(H))
                continue;
            live[i] = true;
            const uint8_t* p = NCX ? in + static_cast<int64_t>(n) * CC * X + static_cast<int64_t>(y) * W + x : in + (static_cast<int64_t>(n) * X + static_cast<int64_t>(y) * W + x) * CC;
#pragma unroll
            for (int c = 0; c < CC; ++c)
                word[i][c] = *reinterpret_cast<const uint32_t*>(p + (NCX ? c * X : static_cast<int64_t>(4 * c)));
        }
        const int32_t xp = x + pbw;
#pragma unroll
        for (int i = 0; i < kQuadRows; ++i)
        {
            const uint32_t row = row0 + i;
            if (row >= rows)
                continue;
            Quad v;
#pragma unroll
            for (int t = 0; t < 4; ++t)
            {
                v.px[t] = fill;
                if (!live[i])
                    continue;
#pragma unroll
                for (int c = 0; c < CC; ++c)
                {
                    const int k = t * CC + c; // byte of the run in [N][H][W][C] data
                    const uint32_t b = NCX ? (word[i][c] >> (8 * t)) & 0xffu : (word[i][k >> 2] >> (8 * (k & 3))) & 0xffu;
                    v.px[t] = (v.px[t] & ~(0xffu << (8 * c))) | (b << (8 * c));
                }
            }
            uint32_t* o = out + static_cast<int64_t>(row) * Wp + xp;
            if (xp >= 0 && xp + 3 < Wp)
                *reinterpret_cast<Quad*>(o) = v;
            else
            {
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (xp + t >= 0 && xp + t < Wp)
                        o[t] = v.px[t];
            }
        }
    }

    int launch_stage_rows(const ConvGeom& g, const RowPack& rp, const void* in, void* staged, const void* zp, int zp_t, hipStream_t s)
    {
        const int64_t rows = g.N * rp.Hp;
        if (rows == 0 || rp.Wp == 0)
            return HIPQ_OK;
        if (g.in[2] % 4 == 0 && (reinterpret_cast<uintptr_t>(in) & 3) == 0 && rows < (1ll << 31) - 64 && getenv("HIPQ_NO_STAGE_QUADS") == nullptr)
        {
            const int64_t first_quad = -((g.pb[2] + 3) / 4);
            const int64_t span = rp.Wp - g.pb[2];                                 // staged pixels from the image's first column on
            const int64_t end_quad = span >= 0 ? (span + 3) / 4 : -((-span) / 4); // ceil(span / 4)
            const int64_t quads = end_quad - first_quad;
            if (quads >= 1 && (quads + 63) / 64 <= 65535 && fits_i32(g.pb[2] + 4 * end_quad))
            {
                const int rows_a_block = 4 * kQuadRows;
                dim3 grid(static_cast<unsigned>((rows + rows_a_block - 1) / rows_a_block), static_cast<unsigned>((quads + 63) / 64));
                const bool ncx = g.data_layout == HIPQ_LAYOUT_NCX;
                auto go = [&](auto kernel) {
                    kernel<<<grid, 256, 0, s>>>(static_cast<const uint8_t*>(in), static_cast<uint32_t*>(staged), static_cast<uint32_t>(rows), static_cast<int32_t>(rp.Hp), static_cast<int32_t>(rp.Wp),
                                                static_cast<int32_t>(g.in[1]), static_cast<int32_t>(g.in[2]), static_cast<int32_t>(g.pb[1]), static_cast<int32_t>(g.pb[2]),
                                                static_cast<int32_t>(first_quad), static_cast<int32_t>(quads), zp, zp_t);
                };
                switch (g.C)
                {
                case 1: ncx ? go(stage_rows_quads_kernel<1, true>) : go(stage_rows_quads_kernel<1, false>); break;
                case 2: ncx ? go(stage_rows_quads_kernel<2, true>) : go(stage_rows_quads_kernel<2, false>); break;
                case 3: ncx ? go(stage_rows_quads_kernel<3, true>) : go(stage_rows_quads_kernel<3, false>); break;
                default: ncx ? go(stage_rows_quads_kernel<4, true>) : go(stage_rows_quads_kernel<4, false>); break;
                }
                return check_launch("stage_rows");
            }
        }
        HIPQ_REQUIRE(rows < (1ll << 31) && (rp.Wp + 255) / 256 <= 65535, "tensor too large for one launch");
        dim3 grid(static_cast<unsigned>((rows + kStageRows - 1) / kStageRows), static_cast<unsigned>((rp.Wp + 255) / 256));
        stage_rows_kernel<<<grid, 256, 0, s>>>(static_cast<const uint8_t*>(in), static_cast<uint32_t*>(staged), static_cast<uint32_t>(rows), static_cast<int32_t>(rp.Hp),
                                               static_cast<int32_t>(rp.Wp), static_cast<int32_t>(g.in[1]), static_cast<int32_t>(g.in[2]), static_cast<int32_t>(g.C),
                                               static_cast<int32_t>(g.pb[1]), static_cast<int32_t>(g.pb[2]), g.data_layout == HIPQ_LAYOUT_NCX ? 1 : 0, zp, zp_t);
        return check_launch("stage_rows");
    }

    int launch_conv_rowpack(const ConvGeom& g, const RowPack& rp, const void* staged, const void* packed, const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s)
    {
        HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(staged) & 15) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0,
                     "MFMA convolution needs 16-byte aligned tensors");
        ConvR xl;
        xl.x = static_cast<const uint8_t*>(staged);
        xl.bytes = static_cast<uint32_t>(g.N * rp.Hp * rp.Wp * 4);
        xl.R = static_cast<int32_t>(g.f[1]);
        xl.S = static_cast<int32_t>(g.f[2]);
        xl.C = static_cast<int32_t>(g.C);
        xl.row_pitch = static_cast<int32_t>(rp.Wp * 4);
        xl.img_pitch = static_cast<int32_t>(rp.Hp * rp.Wp * 4);
        xl.sh_pitch = static_cast<int32_t>(g.st[1] * rp.Wp * 4);
        xl.sw4 = static_cast<int32_t>(g.st[2] * 4);
        xl.Q = static_cast<int32_t>(g.out[2]);
        xl.PQ = static_cast<int32_t>(g.out[1] * g.out[2]);
        xl.by_pq = fast_div(xl.PQ);
        xl.by_q = fast_div(xl.Q);
        const int64_t M = g.N * g.out[1] * g.out[2];
        const int32_t N = static_cast<int32_t>(g.K);
        const int32_t Kred = static_cast<int32_t>(rp.kp);
        const int8_t* w = static_cast<const int8_t*>(packed);
        const int32_t* wsum = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(packed) + align_up(static_cast<size_t>(g.K) * Kred, 256));
        OutMap om{0, N, xl.PQ};
        const int rc = launch_uniform(xl, w, wsum, M, N, Kred, g.data_t == HIPQ_U8 ? 1 : 0, zp, epi, om, out, s, "conv_mfma_i8_32x32x32");
        if (rc == HIPQ_ERR_UNSUPPORTED)
            return fail(HIPQ_ERR_INVALID, "row-packed convolution: output is not an aligned 8-bit channels-last tensor");
        return rc;
    }
}
