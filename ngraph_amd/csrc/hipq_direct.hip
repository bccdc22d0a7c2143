// Direct (one output element per lane) convolution and dot kernels.
//
// These cover every case of the reference kernels -- 1-D to 3-D, any stride / filter dilation /
// data dilation / negative padding, u8 or i8 filters, non-zero zero points, both tensor layouts --
// and are what runs when a shape is not eligible for the MFMA kernels.  They follow
// src/ngraph/runtime/reference/convolution.hpp:102-251 and dot.hpp:93-150 term by term: a tap
// contributes only when it lands on a real input element (not padding, not a data-dilation gap).
#include "hipq_common.h"

namespace hipq
{
    int make_geom(const hipq_conv_desc_t* d, ConvGeom* g)
    {
        HIPQ_REQUIRE(d, "descriptor is null");
        HIPQ_REQUIRE(d->n_spatial >= 1 && d->n_spatial <= HIPQ_MAX_SPATIAL, "n_spatial %d out of range", d->n_spatial);
        HIPQ_REQUIRE(d->N >= 1 && d->C >= 1 && d->K >= 1, "N, C, K must be positive");
        int lead = 3 - d->n_spatial;
        g->N = d->N;
        g->C = d->C;
        g->K = d->K;
        for (int i = 0; i < 3; ++i)
        {
            g->in[i] = g->f[i] = g->out[i] = g->st[i] = g->dl[i] = g->dd[i] = 1;
            g->pb[i] = 0;
        }
        for (int i = 0; i < d->n_spatial; ++i)
        {
            HIPQ_REQUIRE(d->in_sp[i] >= 1 && d->f_sp[i] >= 1 && d->stride[i] >= 1 && d->dilation[i] >= 1 &&
                             d->data_dilation[i] >= 1,
                         "non-positive extent, stride or dilation on spatial axis %d", i);
            int64_t in_eff = (d->in_sp[i] - 1) * d->data_dilation[i] + 1 + d->pad_below[i] + d->pad_above[i];
            int64_t f_eff = (d->f_sp[i] - 1) * d->dilation[i] + 1;
            HIPQ_REQUIRE(in_eff >= f_eff, "window larger than padded data on spatial axis %d", i);
            int64_t o = (in_eff - f_eff) / d->stride[i] + 1;
            HIPQ_REQUIRE(d->out_sp[i] == o, "out_sp[%d] = %lld, inferred %lld", i, (long long)d->out_sp[i], (long long)o);
            g->in[lead + i] = d->in_sp[i];
            g->f[lead + i] = d->f_sp[i];
            g->out[lead + i] = o;
            g->st[lead + i] = d->stride[i];
            g->dl[lead + i] = d->dilation[i];
            g->dd[lead + i] = d->data_dilation[i];
            g->pb[lead + i] = d->pad_below[i];
        }
        g->data_t = d->data_t;
        g->filter_t = d->filter_t;
        g->out_t = d->out_t;
        g->data_layout = d->data_layout;
        g->out_layout = d->out_layout;
        HIPQ_REQUIRE(d->data_layout == HIPQ_LAYOUT_NCX || d->data_layout == HIPQ_LAYOUT_NXC, "bad data layout");
        HIPQ_REQUIRE(d->out_layout == HIPQ_LAYOUT_NCX || d->out_layout == HIPQ_LAYOUT_NXC, "bad out layout");
        return HIPQ_OK;
    }

    __device__ __forceinline__ int64_t
        act_index(int layout, const int64_t* sp, int64_t Cn, int64_t n, int64_t c, int64_t z, int64_t y, int64_t x)
    {
        int64_t s = (z * sp[1] + y) * sp[2] + x;
        int64_t S = sp[0] * sp[1] * sp[2];
        return layout == HIPQ_LAYOUT_NXC ? (n * S + s) * Cn + c : (n * Cn + c) * S + s;
    }

    __global__ __launch_bounds__(256) void conv_direct_kernel(
        ConvGeom g, const void* __restrict__ data, const void* __restrict__ filter, ZeroPoints zp, Epilogue epi, void* out)
    {
        const int64_t total = g.out_count();
        const int32_t dzp = load_zp(zp.data_zp, zp.data_t);
        const int32_t fzp = load_zp(zp.filter_zp, zp.filter_t);
        const EpiRegs er = epi_load(epi);
        int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; t < total; t += step)
        {
            // t enumerates the output in its own memory order, so stores are lane-contiguous
            int64_t n, k, oz, oy, ox, r = t;
            if (g.out_layout == HIPQ_LAYOUT_NXC)
            {
                k = r % g.K;
                r /= g.K;
                ox = r % g.out[2];
                r /= g.out[2];
                oy = r % g.out[1];
                r /= g.out[1];
                oz = r % g.out[0];
                n = r / g.out[0];
            }
            else
            {
                ox = r % g.out[2];
                r /= g.out[2];
                oy = r % g.out[1];
                r /= g.out[1];
                oz = r % g.out[0];
                r /= g.out[0];
                k = r % g.K;
                n = r / g.K;
            }
            int32_t acc = 0;
            for (int64_t fz = 0; fz < g.f[0]; ++fz)
            {
                int64_t pz = oz * g.st[0] + fz * g.dl[0] - g.pb[0];
                if (pz < 0 || pz > (g.in[0] - 1) * g.dd[0] || pz % g.dd[0] != 0)
                    continue;
                for (int64_t fy = 0; fy < g.f[1]; ++fy)
                {
                    int64_t py = oy * g.st[1] + fy * g.dl[1] - g.pb[1];
                    if (py < 0 || py > (g.in[1] - 1) * g.dd[1] || py % g.dd[1] != 0)
                        continue;
                    for (int64_t fx = 0; fx < g.f[2]; ++fx)
                    {
                        int64_t px = ox * g.st[2] + fx * g.dl[2] - g.pb[2];
                        if (px < 0 || px > (g.in[2] - 1) * g.dd[2] || px % g.dd[2] != 0)
                            continue;
                        int64_t di = act_index(g.data_layout, g.in, g.C, n, 0, pz / g.dd[0], py / g.dd[1], px / g.dd[2]);
                        int64_t dstep = g.data_layout == HIPQ_LAYOUT_NXC ? 1 : g.in[0] * g.in[1] * g.in[2];
                        int64_t fi = (((k * g.C) * g.f[0] + fz) * g.f[1] + fy) * g.f[2] + fx;
                        int64_t fstep = g.f[0] * g.f[1] * g.f[2];
                        for (int64_t c = 0; c < g.C; ++c)
                        {
                            int32_t a = load_q(data, g.data_t, di) - dzp;
                            int32_t b = load_q(filter, g.filter_t, fi) - fzp;
                            acc += a * b;
                            di += dstep;
                            fi += fstep;
                        }
                    }
                }
            }
            store_out(out, epi.out_t, t, epi_apply(epi, er, acc, k, t));
        }
    }

    int launch_conv_direct(
        const ConvGeom& g, const void* data, const void* filter, const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s)
    {
        int64_t total = g.out_count();
        int64_t blocks = (total + 255) / 256;
        if (blocks > 1 << 20)
            blocks = 1 << 20;
        conv_direct_kernel<<<static_cast<unsigned>(blocks), 256, 0, s>>>(g, data, filter, zp, epi, out);
        return check_launch("conv_direct");
    }

    __global__ __launch_bounds__(256) void dot_direct_kernel(
        hipq_dot_desc_t d, const void* __restrict__ a, const void* __restrict__ b, ZeroPoints zp, Epilogue epi, void* out)
    {
        const int64_t total = d.M * d.N;
        const int32_t azp = load_zp(zp.data_zp, zp.data_t);
        const int32_t bzp = load_zp(zp.filter_zp, zp.filter_t);
        const EpiRegs er = epi_load(epi);
        int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; t < total; t += step)
        {
            int64_t m = t / d.N, n = t % d.N;
            int64_t bi = d.b_layout == HIPQ_B_NK ? n * d.K : n;
            int64_t bstep = d.b_layout == HIPQ_B_NK ? 1 : d.N;
            int64_t ai = m * d.K;
            int32_t acc = 0;
            for (int64_t k = 0; k < d.K; ++k)
            {
                acc += (load_q(a, d.a_t, ai) - azp) * (load_q(b, d.b_t, bi) - bzp);
                ai += 1;
                bi += bstep;
            }
            store_out(out, epi.out_t, t, epi_apply(epi, er, acc, n, t));
        }
    }

    int launch_dot_direct(
        const hipq_dot_desc_t& d, const void* a, const void* b, const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s)
    {
        int64_t total = d.M * d.N;
        if (total == 0)
            return HIPQ_OK;
        int64_t blocks = (total + 255) / 256;
        if (blocks > 1 << 20)
            blocks = 1 << 20;
        dot_direct_kernel<<<static_cast<unsigned>(blocks), 256, 0, s>>>(d, a, b, zp, epi, out);
        return check_launch("dot_direct");
    }
}
