// Layout helpers: batched 2-D transposes (NCX <-> NXC), filter repacking, row sums.
#include <algorithm>

#include "hipq_common.h"

namespace hipq
{
    typedef int v4i_t __attribute__((ext_vector_type(4)));

    // in [B][R][Cc] -> out [B][Cc][R], elements of EB bytes, through a padded LDS tile
    template <typename T>
    __global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t R, int64_t Cc)
    {
        __shared__ T tile[64][65];
        const int64_t b = blockIdx.z;
        const int64_t r0 = static_cast<int64_t>(blockIdx.y) * 64;
        const int64_t c0 = static_cast<int64_t>(blockIdx.x) * 64;
        const T* src = in + b * R * Cc;
        T* dst = out + b * R * Cc;
        const int tx = threadIdx.x & 63;
        const int ty = threadIdx.x >> 6;
        for (int i = ty; i < 64; i += 4)
        {
            int64_t r = r0 + i, c = c0 + tx;
            if (r < R && c < Cc)
                tile[i][tx] = src[r * Cc + c];
        }
        __syncthreads();
        for (int i = ty; i < 64; i += 4)
        {
            int64_t c = c0 + i, r = r0 + tx;
            if (r < R && c < Cc)
                dst[c * R + r] = tile[tx][i];
        }
    }

    // Byte transpose at memory speed: in [B][R][Cc] -> out [B][Cc][R], R and Cc multiples of 16.
    // A wavefront owns a 64 x 64 byte tile: every lane loads 16 bytes from each of 4 consecutive
    // rows, transposes its four 4x4 byte blocks in registers (8 v_perm_b32 a block), writes the 16
    // resulting dwords -- 4 rows of one column each -- into a [64 columns][17 dwords] LDS tile, and
    // reads back 16 consecutive rows of one column as the 16-byte piece it stores.  Loads and stores
    // are buffer accesses: tile parts beyond the tensor read zeros and are not written.
    __device__ __forceinline__ void transpose4x4(const uint32_t d[4], uint32_t o[4])
    {
        const uint32_t t0 = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u); // d0.b0 d1.b0 d0.b1 d1.b1
        const uint32_t t1 = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u); // d0.b2 d1.b2 d0.b3 d1.b3
        const uint32_t t2 = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u);
        const uint32_t t3 = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
        o[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
        o[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
        o[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
        o[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
    }

    typedef int v4t __attribute__((ext_vector_type(4)));

    // tiles_c wavefront tiles side by side along the columns, 4 / tiles_c along the rows
    __global__ __launch_bounds__(256) void transpose_bytes_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, int32_t R, int32_t Cc, int32_t tiles_c, uint32_t bytes)
    {
        __shared__ uint32_t tile[4][64][17];
        const int wave = threadIdx.x >> 6;
        const int t = threadIdx.x & 63;
        const int tc = wave % tiles_c, tr = wave / tiles_c;
        const int r0 = (static_cast<int>(blockIdx.y) * (4 / tiles_c) + tr) * 64;
        const int c0 = (static_cast<int>(blockIdx.x) * tiles_c + tc) * 64;
        const uint32_t plane = static_cast<uint32_t>(R) * static_cast<uint32_t>(Cc);
        const __amdgpu_buffer_rsrc_t irs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(in) + static_cast<size_t>(blockIdx.z) * plane, 0, plane, 0x00020000);
        const __amdgpu_buffer_rsrc_t ors = __builtin_amdgcn_make_buffer_rsrc(out + static_cast<size_t>(blockIdx.z) * plane, 0, plane, 0x00020000);
        constexpr int32_t oob = static_cast<int32_t>(0x80000000u);
        (void)bytes;
        {
            const int rg = t >> 2, cb = t & 3; // rows 4rg..4rg+3, columns 16cb..16cb+15 of the tile
            v4t l[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                const int r = r0 + 4 * rg + i, c = c0 + 16 * cb;
                l[i] = __builtin_amdgcn_raw_buffer_load_b128(irs, (r < R && c < Cc) ? r * Cc + c : oob, 0, 0);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const uint32_t d[4] = {static_cast<uint32_t>(l[0][q]), static_cast<uint32_t>(l[1][q]), static_cast<uint32_t>(l[2][q]), static_cast<uint32_t>(l[3][q])};
                uint32_t o[4];
                transpose4x4(d, o);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    tile[wave][16 * cb + 4 * q + j][rg] = o[j];
            }
        }
        // the tile is private to the wavefront and its LDS accesses complete in order: no barrier
        {
#pragma unroll
            for (int it = 0; it < 4; ++it)
            {
                const int col = it * 16 + (t >> 2), q = t & 3;
                const v4t v = v4t{static_cast<int>(tile[wave][col][4 * q]), static_cast<int>(tile[wave][col][4 * q + 1]), static_cast<int>(tile[wave][col][4 * q + 2]),
                                  static_cast<int>(tile[wave][col][4 * q + 3])};
                const int c = c0 + col, r = r0 + 16 * q;
                __builtin_amdgcn_raw_buffer_store_b128(v, ors, (c < Cc && r < R) ? c * R + r : oob, 0, 0);
            }
        }
    }

    int launch_transpose(const void* in, void* out, int64_t B, int64_t R, int64_t Cc, int elem_bytes, hipStream_t s)
    {
        if (B == 0 || R == 0 || Cc == 0)
            return HIPQ_OK;
        HIPQ_REQUIRE(in && out, "null tensor pointer");
        HIPQ_REQUIRE(B <= 65535, "batch %lld beyond 65535", (long long)B);
        if (elem_bytes == 1 && R % 16 == 0 && Cc % 16 == 0 && R * Cc < (1ll << 31) && (reinterpret_cast<uintptr_t>(in) & 15) == 0 &&
            (reinterpret_cast<uintptr_t>(out) & 15) == 0)
        {
            const int tiles_c = Cc > 128 ? 4 : (Cc > 64 ? 2 : 1);
            const int64_t gx = (Cc + 64 * tiles_c - 1) / (64 * tiles_c), gy = (R + 64 * (4 / tiles_c) - 1) / (64 * (4 / tiles_c));
            if (gy <= 65535)
            {
                dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy), static_cast<unsigned>(B));
                transpose_bytes_kernel<<<grid, 256, 0, s>>>(static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), static_cast<int32_t>(R), static_cast<int32_t>(Cc),
                                                           tiles_c, 0u);
                return check_launch("transpose_bytes");
            }
        }
        dim3 grid(static_cast<unsigned>((Cc + 63) / 64), static_cast<unsigned>((R + 63) / 64), static_cast<unsigned>(B));
        HIPQ_REQUIRE((R + 63) / 64 <= 65535, "extent too large for the transpose grid");
        if (elem_bytes == 1)
            transpose_kernel<uint8_t><<<grid, 256, 0, s>>>(static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), R, Cc);
        else if (elem_bytes == 4)
            transpose_kernel<uint32_t><<<grid, 256, 0, s>>>(static_cast<const uint32_t*>(in), static_cast<uint32_t*>(out), R, Cc);
        else
            return fail(HIPQ_ERR_UNSUPPORTED, "transpose of %d-byte elements", elem_bytes);
        return check_launch("transpose");
    }

    // sums[r] = sum_c w[r][c] for i8 rows; one wavefront per row
    __global__ __launch_bounds__(256) void row_sums_i8_kernel(const int8_t* __restrict__ w, int64_t rows, int64_t cols, int32_t* sums)
    {
        const int lane = threadIdx.x & 63;
        const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
        if (row >= rows)
            return;
        const int8_t* p = w + row * cols;
        int32_t acc = 0;
        for (int64_t c = lane; c < cols; c += 64)
            acc += p[c];
        for (int off = 32; off > 0; off >>= 1)
            acc += __shfl_down(acc, off, 64);
        if (lane == 0)
            sums[row] = acc;
    }

    int launch_row_sums_i8(const void* w, int64_t rows, int64_t cols, int32_t* sums, hipStream_t s)
    {
        if (rows == 0)
            return HIPQ_OK;
        row_sums_i8_kernel<<<static_cast<unsigned>((rows + 3) / 4), 256, 0, s>>>(static_cast<const int8_t*>(w), rows, cols, sums);
        return check_launch("row_sums_i8");
    }

    // weights [N][K] -> fragment order of v_mfma_i32_16x16x64_i8's B operand: the 1 KB block of
    // (column block cb, 64-byte reduction step ks) holds, at 16 * lane, what lane (column lane % 16,
    // chunk lane / 16) feeds the instruction: bytes ks * 64 + 16 * (lane / 16) ... of row cb * 16 +
    // lane % 16 (zeros beyond N).  A wavefront then fetches a fragment as 1 KB of contiguous memory
    // -- eight whole cache lines, consecutive lanes in one line -- where the row-major matrix makes
    // consecutive lanes touch sixteen different lines.
    __global__ __launch_bounds__(256) void pack_dot_fragments_kernel(const int8_t* __restrict__ w, int64_t N, int64_t K, v4i_t* __restrict__ frag)
    {
        const int64_t steps = K >> 6;
        const int64_t total = ((N + 15) >> 4) * steps * 64;
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < total; i += stride)
        {
            const int lane = static_cast<int>(i & 63);
            const int64_t blk = i >> 6;
            const int64_t cb = blk / steps, ks = blk - cb * steps;
            const int64_t n = cb * 16 + (lane & 15);
            v4i_t v = {0, 0, 0, 0};
            if (n < N)
                v = *reinterpret_cast<const v4i_t*>(w + n * K + ks * 64 + (lane >> 4) * 16);
            frag[i] = v;
        }
    }

    int launch_pack_dot_fragments(const void* w_nk, int64_t N, int64_t K, void* frag, hipStream_t s)
    {
        const int64_t total = ((N + 15) / 16) * (K / 64) * 64;
        if (total == 0)
            return HIPQ_OK;
        const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((total + 255) / 256, 8192));
        pack_dot_fragments_kernel<<<blocks, 256, 0, s>>>(static_cast<const int8_t*>(w_nk), N, K, static_cast<v4i_t*>(frag));
        return check_launch("pack_dot_fragments");
    }

    // filter [K][C][taps] -> packed [K][taps][Cp], channels C .. Cp-1 zero
    __global__ __launch_bounds__(256) void pack_filter_kernel(
        const int8_t* __restrict__ f, int8_t* __restrict__ p, int64_t K, int64_t Cc, int64_t Cp, int64_t taps)
    {
        int64_t total = K * Cp * taps;
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < total; i += step)
        {
            int64_t c = i % Cp;
            int64_t t = (i / Cp) % taps;
            int64_t k = i / (Cp * taps);
            p[i] = c < Cc ? f[(k * Cc + c) * taps + t] : static_cast<int8_t>(0);
        }
    }

    // filter [K][C][R][S] -> row-packed [K][kp]: byte r * 32 + s * 4 + c holds tap (r, s) of channel c,
    // everything else (taps s >= S, channels c >= C, the tail up to kp) is zero
    __global__ __launch_bounds__(256) void pack_filter_rows_kernel(const int8_t* __restrict__ f, int8_t* __restrict__ p, int64_t K, int32_t Cc, int32_t R, int32_t S, int32_t kp)
    {
        const int64_t total = K * kp;
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < total; i += step)
        {
            const int64_t k = i / kp;
            const int32_t b = static_cast<int32_t>(i - k * kp);
            const int32_t r = b >> 5, s = (b >> 2) & 7, c = b & 3;
            p[i] = (r < R && s < S && c < Cc) ? f[((k * Cc + c) * R + r) * S + s] : static_cast<int8_t>(0);
        }
    }

    // [N][C][X] or [N][X][C] bytes -> [N][X][16] with the channels C .. 15 holding the data zero point
    // (they meet zero weights; as the zero point they also vanish on the exact path for a non-zero
    // filter zero point); one pixel a lane, one 16-byte store
    __global__ __launch_bounds__(256) void pad_channels_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, int64_t pixels, int64_t X, int32_t Cc, int32_t in_ncx,
                                                               const void* zp, int32_t zp_t)
    {
        const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
        if (i >= pixels)
            return;
        const int64_t n = i / X, x = i - n * X;
        const uint32_t fill = (static_cast<uint32_t>(load_zp(zp, zp_t)) & 0xffu) * 0x01010101u;
        uint32_t w[4] = {fill, fill, fill, fill};
        for (int c = 0; c < Cc; ++c)
            w[c >> 2] &= ~(0xffu << (8 * (c & 3)));
        for (int c = 0; c < Cc; ++c)
        {
            const uint32_t b = in_ncx ? in[(n * Cc + c) * X + x] : in[i * Cc + c];
            w[c >> 2] |= b << (8 * (c & 3));
        }
        reinterpret_cast<uint4*>(out)[i] = make_uint4(w[0], w[1], w[2], w[3]);
    }

    int launch_pad_channels(const void* in, void* out, int64_t N, int64_t X, int64_t Cc, bool in_ncx, const void* zp, int zp_t, hipStream_t s)
    {
        const int64_t pixels = N * X;
        if (pixels == 0)
            return HIPQ_OK;
        HIPQ_REQUIRE(Cc >= 1 && Cc < 16, "channel padding takes fewer than 16 channels");
        HIPQ_REQUIRE((pixels + 255) / 256 < (1ll << 31), "tensor too large for one launch");
        pad_channels_kernel<<<static_cast<unsigned>((pixels + 255) / 256), 256, 0, s>>>(static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), pixels, X, static_cast<int32_t>(Cc),
                                                                                       in_ncx ? 1 : 0, zp, zp_t);
        return check_launch("pad_channels");
    }

    // Channels-last data -> the [M][taps * C] matrix of a convolution's receptive fields (M = images x
    // output pixels), 16 bytes a lane; taps in the padding hold the data zero point, which
    // contributes nothing.  Only for the few-row case (M <= 64), where the matrix is small and the
    // weight-streaming GEMM kernels beat the tiled ones by far.
    __global__ __launch_bounds__(256) void im2col_nxc_kernel(const uint8_t* __restrict__ x, uint8_t* __restrict__ a, ConvGeom g, int32_t M, int32_t chunks_per_row, const void* zp, int32_t zp_t)
    {
        const int32_t i = static_cast<int32_t>(blockIdx.x) * 256 + threadIdx.x;
        if (i >= M * chunks_per_row)
            return;
        const int32_t m = i / chunks_per_row;
        const int32_t kbyte = (i - m * chunks_per_row) * 16;
        const int32_t Cc = static_cast<int32_t>(g.C), S = static_cast<int32_t>(g.f[2]);
        const int32_t tap = kbyte / Cc, c = kbyte - tap * Cc;
        const int32_t r = tap / S, s = tap - r * S;
        const int32_t PQ = static_cast<int32_t>(g.out[1] * g.out[2]), Q = static_cast<int32_t>(g.out[2]);
        const int32_t n = m / PQ, rem = m - n * PQ;
        const int32_t p = rem / Q, q = rem - p * Q;
        const int32_t iy = p * static_cast<int32_t>(g.st[1]) - static_cast<int32_t>(g.pb[1]) + r * static_cast<int32_t>(g.dl[1]);
        const int32_t ix = q * static_cast<int32_t>(g.st[2]) - static_cast<int32_t>(g.pb[2]) + s * static_cast<int32_t>(g.dl[2]);
        uint4 v;
        if (static_cast<uint32_t>(iy) < static_cast<uint32_t>(g.in[1]) && static_cast<uint32_t>(ix) < static_cast<uint32_t>(g.in[2]))
            v = *reinterpret_cast<const uint4*>(x + ((static_cast<int64_t>(n) * g.in[1] + iy) * g.in[2] + ix) * Cc + c);
        else
        {
            const uint32_t fill = (static_cast<uint32_t>(load_zp(zp, zp_t)) & 0xffu) * 0x01010101u;
            v = make_uint4(fill, fill, fill, fill);
        }
        reinterpret_cast<uint4*>(a)[i] = v;
    }

    int launch_im2col_nxc(const ConvGeom& g, const void* x_nxc, void* a, const void* zp, int zp_t, hipStream_t s)
    {
        const int64_t M = g.N * g.out[1] * g.out[2];
        const int64_t kred = g.C * g.taps();
        HIPQ_REQUIRE(g.C % 16 == 0 && M * kred < (1ll << 31), "im2col takes multiples of 16 channels and matrices below 2 GiB");
        const int64_t lanes = M * (kred / 16);
        if (lanes == 0)
            return HIPQ_OK;
        im2col_nxc_kernel<<<static_cast<unsigned>((lanes + 255) / 256), 256, 0, s>>>(static_cast<const uint8_t*>(x_nxc), static_cast<uint8_t*>(a), g, static_cast<int32_t>(M),
                                                                                  static_cast<int32_t>(kred / 16), zp, zp_t);
        return check_launch("im2col_nxc");
    }

    // Fewer than 16 input channels (a network's first layer): the MFMA kernels take the layer with the
    // channels padded to 16 -- zero weights in the packed filter, a padded copy of the data
    bool conv_pad_eligible(const ConvGeom& g, ConvGeom* padded)
    {
        if (g.C >= 16 || g.C < 1)
            return false;
        ConvGeom p = g;
        p.C = 16;
        p.data_layout = HIPQ_LAYOUT_NXC;
        if (!conv_mfma_eligible(p))
            return false;
        if (padded)
            *padded = p;
        return true;
    }
}

using namespace hipq;

extern "C" {

int hipq_transpose_ncx_to_nxc(const void* in, void* out, int64_t N, int64_t C, int64_t X, int32_t elem_bytes, void* stream)
{
    HIPQ_REQUIRE(N >= 0 && C >= 0 && X >= 0, "negative extent");
    return launch_transpose(in, out, N, C, X, elem_bytes, as_stream(stream));
}

int hipq_transpose_nxc_to_ncx(const void* in, void* out, int64_t N, int64_t C, int64_t X, int32_t elem_bytes, void* stream)
{
    HIPQ_REQUIRE(N >= 0 && C >= 0 && X >= 0, "negative extent");
    return launch_transpose(in, out, N, X, C, elem_bytes, as_stream(stream));
}

size_t hipq_conv_packed_filter_bytes(const hipq_conv_desc_t* desc)
{
    ConvGeom g;
    if (make_geom(desc, &g) != HIPQ_OK)
        return 0;
    RowPack rp;
    if (conv_rowpack_eligible(g, &rp))
        return align_up(static_cast<size_t>(g.K * rp.kp), 256) + static_cast<size_t>(g.K) * sizeof(int32_t);
    if (!conv_mfma_eligible(g) && !conv_pad_eligible(g, &g))
        return 0;
    size_t w = align_up(static_cast<size_t>(g.K * g.C * g.taps()), 256);
    return w + static_cast<size_t>(g.K) * sizeof(int32_t);
}

int hipq_conv_pack_filter(const hipq_conv_desc_t* desc, const void* filter, void* packed, void* stream)
{
    ConvGeom g;
    int rc = make_geom(desc, &g);
    if (rc)
        return rc;
    const int64_t src_c = g.C;
    RowPack rp;
    if (conv_rowpack_eligible(g, &rp))
    {
        HIPQ_REQUIRE(filter && packed, "null pointer");
        hipStream_t s = as_stream(stream);
        const int64_t total = g.K * rp.kp;
        int64_t blocks = (total + 255) / 256;
        if (blocks > 65536)
            blocks = 65536;
        pack_filter_rows_kernel<<<static_cast<unsigned>(blocks), 256, 0, s>>>(static_cast<const int8_t*>(filter), static_cast<int8_t*>(packed), g.K, static_cast<int32_t>(g.C),
                                                                              static_cast<int32_t>(g.f[1]), static_cast<int32_t>(g.f[2]), static_cast<int32_t>(rp.kp));
        rc = check_launch("pack_filter_rows");
        if (rc)
            return rc;
        int32_t* sums = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(packed) + align_up(static_cast<size_t>(total), 256));
        return launch_row_sums_i8(packed, g.K, rp.kp, sums, s);
    }
    if (!conv_mfma_eligible(g) && !conv_pad_eligible(g, &g))
        return fail(HIPQ_ERR_UNSUPPORTED, "shape is not eligible for the MFMA path (hipq_conv_packed_filter_bytes is 0)");
    HIPQ_REQUIRE(filter && packed, "null pointer");
    hipStream_t s = as_stream(stream);
    int64_t total = g.K * g.C * g.taps();
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536)
        blocks = 65536;
    pack_filter_kernel<<<static_cast<unsigned>(blocks), 256, 0, s>>>(
        static_cast<const int8_t*>(filter), static_cast<int8_t*>(packed), g.K, src_c, g.C, g.taps());
    rc = check_launch("pack_filter");
    if (rc)
        return rc;
    int32_t* sums = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(packed) + align_up(static_cast<size_t>(total), 256));
    return launch_row_sums_i8(packed, g.K, g.C * g.taps(), sums, s);
}
}
