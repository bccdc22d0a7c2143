// Layout helpers: batched 2-D transposes (NCX <-> NXC), filter repacking, row sums.
#include "hipq_common.h"

namespace hipq
{
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

    int launch_transpose(const void* in, void* out, int64_t B, int64_t R, int64_t Cc, int elem_bytes, hipStream_t s)
    {
        if (B == 0 || R == 0 || Cc == 0)
            return HIPQ_OK;
        HIPQ_REQUIRE(in && out, "null tensor pointer");
        HIPQ_REQUIRE(B <= 65535, "batch %lld beyond 65535", (long long)B);
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

    // filter [K][C][taps] -> packed [K][taps][C]
    __global__ __launch_bounds__(256) void pack_filter_kernel(
        const int8_t* __restrict__ f, int8_t* __restrict__ p, int64_t K, int64_t Cc, int64_t taps)
    {
        int64_t total = K * Cc * taps;
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < total; i += step)
        {
            int64_t c = i % Cc;
            int64_t t = (i / Cc) % taps;
            int64_t k = i / (Cc * taps);
            p[i] = f[(k * Cc + c) * taps + t];
        }
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
    if (make_geom(desc, &g) != HIPQ_OK || !conv_mfma_eligible(g))
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
    if (!conv_mfma_eligible(g))
        return fail(HIPQ_ERR_UNSUPPORTED, "shape is not eligible for the MFMA path (hipq_conv_packed_filter_bytes is 0)");
    HIPQ_REQUIRE(filter && packed, "null pointer");
    hipStream_t s = as_stream(stream);
    int64_t total = g.K * g.C * g.taps();
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536)
        blocks = 65536;
    pack_filter_kernel<<<static_cast<unsigned>(blocks), 256, 0, s>>>(
        static_cast<const int8_t*>(filter), static_cast<int8_t*>(packed), g.K, g.C, g.taps());
    rc = check_launch("pack_filter");
    if (rc)
        return rc;
    int32_t* sums = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(packed) + align_up(static_cast<size_t>(total), 256));
    return launch_row_sums_i8(packed, g.K, g.C * g.taps(), sums, s);
}
}
