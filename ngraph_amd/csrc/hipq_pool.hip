// MaxPool / AvgPool / Concat: the integer glue between the quantized convolutions of a network.
// One output element per lane; channels-last tensors put consecutive lanes on consecutive
// channels of a pixel, NCHW tensors on consecutive pixels of a row -- coalesced either way.
#include <cmath>
#include <limits>

#include "hipq_common.h"

namespace hipq
{
    struct PoolGeom
    {
        int64_t N, C;
        int64_t in[3], win[3], st[3], pb[3], out[3];
        int32_t nxc;
        int32_t include_padding;
        int64_t count;
    };

    template <typename T, bool AVG>
    __global__ __launch_bounds__(256) void pool_kernel(PoolGeom g, const T* __restrict__ in, T* __restrict__ out)
    {
        const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
        if (i >= g.count)
            return;
        // flat output index -> (n, c, o0, o1, o2) in the tensor's layout
        int64_t n, c, o[3];
        int64_t t = i;
        if (g.nxc)
        {
            c = t % g.C;
            t /= g.C;
        }
        o[2] = t % g.out[2];
        t /= g.out[2];
        o[1] = t % g.out[1];
        t /= g.out[1];
        o[0] = t % g.out[0];
        t /= g.out[0];
        if (!g.nxc)
        {
            c = t % g.C;
            t /= g.C;
        }
        n = t;
        const int64_t in_sp = g.in[0] * g.in[1] * g.in[2];
        // src/ngraph/runtime/reference/max_pool.hpp:209 : lowest(); avg_pool.hpp:216 : T result = 0
        T best = std::numeric_limits<T>::lowest();
        T sum = 0;
        int64_t cnt = 0;
        for (int64_t w0 = 0; w0 < g.win[0]; ++w0)
            for (int64_t w1 = 0; w1 < g.win[1]; ++w1)
                for (int64_t w2 = 0; w2 < g.win[2]; ++w2)
                {
                    const int64_t y0 = o[0] * g.st[0] + w0 - g.pb[0];
                    const int64_t y1 = o[1] * g.st[1] + w1 - g.pb[1];
                    const int64_t y2 = o[2] * g.st[2] + w2 - g.pb[2];
                    const bool inb = y0 >= 0 && y0 < g.in[0] && y1 >= 0 && y1 < g.in[1] && y2 >= 0 && y2 < g.in[2];
                    if (inb)
                    {
                        const int64_t sp = (y0 * g.in[1] + y1) * g.in[2] + y2;
                        const T v = g.nxc ? in[(n * in_sp + sp) * g.C + c] : in[(n * g.C + c) * in_sp + sp];
                        if (AVG)
                        {
                            sum = static_cast<T>(sum + v); // the reference sums in T: 8-bit sums wrap
                            ++cnt;
                        }
                        else
                            best = v > best ? v : best;
                    }
                    else if (AVG && g.include_padding)
                        ++cnt;
                }
        if (AVG)
        {
            // avg_pool.hpp:238-246 : nearbyint(float(sum) / count) for 8-bit types, plain division else
            if (sizeof(T) == 1)
                out[i] = static_cast<T>(rintf(static_cast<float>(sum) / static_cast<float>(static_cast<uint64_t>(cnt))));
            else
                out[i] = static_cast<T>(sum / static_cast<T>(static_cast<uint64_t>(cnt)));
        }
        else
            out[i] = best;
    }

    // out[(o * total + offset + e) * inner + j] = in[(o * extent + e) * inner + j], one byte group per lane
    template <typename T>
    __global__ __launch_bounds__(256) void concat_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t count, int64_t piece, int64_t total, int64_t offset)
    {
        const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
        if (i >= count)
            return;
        const int64_t o = i / piece;
        const int64_t r = i - o * piece;
        out[o * total + offset + r] = in[i];
    }

    template <typename T>
    static int launch_pool(const PoolGeom& g, int op, const void* in, void* out, hipStream_t s)
    {
        const unsigned grid = static_cast<unsigned>((g.count + 255) / 256);
        if (op == HIPQ_POOL_AVG)
            pool_kernel<T, true><<<grid, 256, 0, s>>>(g, static_cast<const T*>(in), static_cast<T*>(out));
        else
            pool_kernel<T, false><<<grid, 256, 0, s>>>(g, static_cast<const T*>(in), static_cast<T*>(out));
        return check_launch(op == HIPQ_POOL_AVG ? "avg_pool" : "max_pool");
    }
}

using namespace hipq;

extern "C" {

int hipq_pool_infer_output(hipq_pool_desc_t* d)
{
    HIPQ_REQUIRE(d, "descriptor is null");
    HIPQ_REQUIRE(d->n_spatial >= 1 && d->n_spatial <= HIPQ_MAX_SPATIAL, "n_spatial %d out of range", d->n_spatial);
    for (int i = 0; i < d->n_spatial; ++i)
    {
        HIPQ_REQUIRE(d->in_sp[i] >= 1 && d->window[i] >= 1 && d->stride[i] >= 1 && d->pad_below[i] >= 0 && d->pad_above[i] >= 0,
                     "non-positive extent, window or stride, or negative padding on spatial axis %d", i);
        const int64_t padded = d->in_sp[i] + d->pad_below[i] + d->pad_above[i];
        HIPQ_REQUIRE(padded >= d->window[i], "window larger than padded data on spatial axis %d", i);
        d->out_sp[i] = (padded - d->window[i]) / d->stride[i] + 1;
    }
    return HIPQ_OK;
}

int hipq_pool(const hipq_pool_desc_t* d, const void* in, void* out, void* stream)
{
    HIPQ_REQUIRE(d, "descriptor is null");
    hipq_pool_desc_t chk = *d;
    int rc = hipq_pool_infer_output(&chk);
    if (rc)
        return rc;
    HIPQ_REQUIRE(d->op == HIPQ_POOL_MAX || d->op == HIPQ_POOL_AVG, "pool op %d unknown", d->op);
    HIPQ_REQUIRE(d->layout == HIPQ_LAYOUT_NCX || d->layout == HIPQ_LAYOUT_NXC, "layout %d unknown", d->layout);
    HIPQ_REQUIRE(d->N >= 0 && d->C >= 0, "negative extent");
    PoolGeom g;
    g.N = d->N;
    g.C = d->C;
    g.nxc = d->layout == HIPQ_LAYOUT_NXC;
    g.include_padding = d->include_padding;
    // normalise to three spatial axes, leading ones of extent 1
    const int lead = 3 - d->n_spatial;
    for (int i = 0; i < 3; ++i)
    {
        const bool real = i >= lead;
        g.in[i] = real ? d->in_sp[i - lead] : 1;
        g.win[i] = real ? d->window[i - lead] : 1;
        g.st[i] = real ? d->stride[i - lead] : 1;
        g.pb[i] = real ? d->pad_below[i - lead] : 0;
        g.out[i] = real ? chk.out_sp[i - lead] : 1;
        HIPQ_REQUIRE(!real || d->out_sp[i - lead] == chk.out_sp[i - lead], "out_sp[%d] does not match the window geometry", i - lead);
    }
    g.count = g.N * g.C * g.out[0] * g.out[1] * g.out[2];
    if (g.count == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && out, "null tensor pointer");
    HIPQ_REQUIRE((g.count + 255) / 256 < (1ll << 31), "tensor too large for one launch");
    if (d->op == HIPQ_POOL_AVG)
    {
        // a window that sees neither data nor counted padding has no average: the reference throws
        for (int i = 0; i < 3; ++i)
            HIPQ_REQUIRE(d->include_padding || (g.pb[i] < g.win[i] && (g.out[i] - 1) * g.st[i] - g.pb[i] < g.in[i]),
                         "AvgPool window wholly inside the padding (elements == 0)");
    }
    hipStream_t s = as_stream(stream);
    switch (d->dtype)
    {
    case HIPQ_U8: return launch_pool<uint8_t>(g, d->op, in, out, s);
    case HIPQ_I8: return launch_pool<int8_t>(g, d->op, in, out, s);
    case HIPQ_F32: return launch_pool<float>(g, d->op, in, out, s);
    case HIPQ_I32:
        if (d->op == HIPQ_POOL_MAX)
            return launch_pool<int32_t>(g, d->op, in, out, s);
        return fail(HIPQ_ERR_UNSUPPORTED, "AvgPool on i32 is not supported");
    default: return fail(HIPQ_ERR_UNSUPPORTED, "pooling on dtype %d", d->dtype);
    }
}

int hipq_concat(int32_t elem_bytes,
                int32_t n_inputs,
                const void* const* inputs,
                const int64_t* extents,
                int64_t outer,
                int64_t inner,
                void* out,
                void* stream)
{
    HIPQ_REQUIRE(n_inputs >= 0 && outer >= 0 && inner >= 0, "negative extent");
    HIPQ_REQUIRE(elem_bytes == 1 || elem_bytes == 4 || elem_bytes == 8, "concat of %d-byte elements", elem_bytes);
    HIPQ_REQUIRE(n_inputs == 0 || (inputs && extents), "null input table");
    int64_t total = 0;
    for (int i = 0; i < n_inputs; ++i)
    {
        HIPQ_REQUIRE(extents[i] >= 0, "negative extent of input %d", i);
        total += extents[i];
    }
    hipStream_t s = as_stream(stream);
    int64_t offset = 0;
    for (int i = 0; i < n_inputs; ++i)
    {
        const int64_t piece = extents[i] * inner;
        const int64_t count = outer * piece;
        if (count > 0)
        {
            HIPQ_REQUIRE(inputs[i] && out, "null tensor pointer");
            HIPQ_REQUIRE((count + 255) / 256 < (1ll << 31), "tensor too large for one launch");
            const unsigned grid = static_cast<unsigned>((count + 255) / 256);
            if (elem_bytes == 1)
                concat_kernel<uint8_t><<<grid, 256, 0, s>>>(static_cast<const uint8_t*>(inputs[i]), static_cast<uint8_t*>(out), count, piece, total * inner, offset * inner);
            else if (elem_bytes == 4)
                concat_kernel<uint32_t><<<grid, 256, 0, s>>>(static_cast<const uint32_t*>(inputs[i]), static_cast<uint32_t*>(out), count, piece, total * inner, offset * inner);
            else
                concat_kernel<uint64_t><<<grid, 256, 0, s>>>(static_cast<const uint64_t*>(inputs[i]), static_cast<uint64_t*>(out), count, piece, total * inner, offset * inner);
            int rc = check_launch("concat");
            if (rc)
                return rc;
        }
        offset += extents[i];
    }
    return HIPQ_OK;
}
}
