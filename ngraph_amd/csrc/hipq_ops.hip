// Entry points of the quantized convolution / dot family: argument checks, choice between the
// MFMA kernels and the direct kernels, layout conversion through the device workspace.
#include <cstdlib>

#include <cstring>

#include "hipq_common.h"

namespace hipq
{
    static bool is_quant8(int t) { return t == HIPQ_U8 || t == HIPQ_I8; }

    static int check_conv_types(const ConvGeom& g, bool fused)
    {
        // INTERPRETER combinations: int_executable.hpp:1461-1549 (data is u8 there); i8 data is
        // accepted as well because the oneDNN-backed fused ops take it.
        if (!is_quant8(g.data_t) || !is_quant8(g.filter_t))
            return fail(HIPQ_ERR_UNSUPPORTED, "data and filter must be u8 or i8");
        if (!is_quant8(g.out_t) && g.out_t != HIPQ_I32)
            return fail(HIPQ_ERR_UNSUPPORTED, "convolution output must be i8, u8 or i32");
        if (fused && g.filter_t != HIPQ_I8)
            return fail(HIPQ_ERR_UNSUPPORTED, "fused convolutions take i8 filters");
        return HIPQ_OK;
    }

    // Runs the convolution with whatever layouts the descriptor names.
    static int run_conv(const ConvGeom& g,
                        const void* data,
                        const void* filter,
                        const void* packed,
                        const ZeroPoints& zp,
                        Epilogue epi,
                        void* out,
                        hipStream_t s)
    {
        // the MFMA kernels have no fused-policy instantiation with int32 output (no nGraph op asks for one)
        RowPack rp;
        // a first layer the band kernel takes whole: it reads the [N][C][H][W] bytes itself
        if (packed && (reinterpret_cast<uintptr_t>(data) & 3) == 0 && conv_rowpack_eligible(g, &rp) && conv_stem_eligible(g, epi, zp, nullptr))
            return launch_conv_stem(g, data, packed, zp, epi, nullptr, out, s);
        if (packed && conv_rowpack_eligible(g, &rp))
        {
            // a first layer's three or four channels: a copy with the padding materialised, whose
            // filter rows are single 32-byte runs, then the tile kernel that loads straight into LDS
            void* ws = nullptr;
            int rc = workspace(align_up(static_cast<size_t>(g.N * rp.Hp * rp.Wp * 4), 256), s, &ws);
            if (rc)
                return rc;
            rc = launch_stage_rows(g, rp, data, ws, zp.data_zp, zp.data_t, s);
            if (rc)
                return rc;
            return launch_conv_rowpack(g, rp, ws, packed, zp, epi, out, s);
        }
        ConvGeom padded;
        if (packed && !conv_mfma_eligible(g) && conv_pad_eligible(g, &padded) && !(epi.mode == EPI_FUSED && g.out_t == HIPQ_I32))
        {
            // a first layer's few channels: a 16-channel channels-last copy, then the MFMA kernel
            void* ws = nullptr;
            const int64_t in_sp = g.in[1] * g.in[2];
            int rc = workspace(align_up(static_cast<size_t>(g.N * in_sp * 16), 256), s, &ws);
            if (rc)
                return rc;
            rc = launch_pad_channels(data, ws, g.N, in_sp, g.C, g.data_layout == HIPQ_LAYOUT_NCX, zp.data_zp, zp.data_t, s);
            if (rc)
                return rc;
            return launch_conv_mfma(padded, ws, packed, zp, epi, out, g.out_layout == HIPQ_LAYOUT_NCX && g.K > 1, s);
        }
        if (!packed || !conv_mfma_eligible(g) || (epi.mode == EPI_FUSED && g.out_t == HIPQ_I32))
            return launch_conv_direct(g, data, filter, zp, epi, out, s);

        // layers bound by HBM traffic that widen 64 channels: weights in registers, loads a tile ahead
        if (conv_pw64_eligible(g, epi, zp))
            return launch_conv_pw64(g, data, packed, epi, out, s);

        // 3x3 layers over 64 channels with an NCHW output keep their filter in registers and read the
        // input in whichever layout it has: no transposition, no scratch
        if (conv_regw_eligible(g, g.out_layout == HIPQ_LAYOUT_NCX && g.K > 1))
            return launch_conv_regw(g, data, packed, zp, epi, out, true, s);

        // The other kernels read channels-last data; an NCHW input is transposed through the workspace.
        // The output is written directly in either layout (sum_in is indexed like the output).
        // A layer with few output pixels in all (M <= 64: the deepest layers of a network at batch 1)
        // is a skinny GEMM over its receptive-field matrix [M][taps * C] -- the data itself for a 1x1
        // stride-1 filter, an im2col copy in the workspace otherwise -- and takes the weight-streaming
        // GEMM kernels, which spread the filter over every CU where tiles of M would fill a few.
        const int64_t in_sp = g.in[1] * g.in[2];
        const bool tr_in = g.data_layout == HIPQ_LAYOUT_NCX && g.C > 1;
        const int64_t M = g.N * g.out[1] * g.out[2];
        const int64_t kred = g.C * g.taps();
        const bool pointwise = g.taps() == 1 && g.st[1] == 1 && g.st[2] == 1 && g.pb[1] == 0 && g.pb[2] == 0 && g.out[1] == g.in[1] && g.out[2] == g.in[2];
        const bool as_gemm = !(g.out_layout == HIPQ_LAYOUT_NCX && g.K > 1) && M <= 64 && kred % 64 == 0 && kred >= 256 && M * kred < (1ll << 31) &&
                             g.filter_t == HIPQ_I8 && getenv("HIPQ_NO_SKINNY") == nullptr;
        const size_t tr_bytes = tr_in ? align_up(static_cast<size_t>(g.in_count()), 256) : 0;
        const size_t col_bytes = (as_gemm && !pointwise) ? align_up(static_cast<size_t>(M * kred), 256) : 0;
        const void* x = data;
        uint8_t* ws = nullptr;
        if (tr_bytes + col_bytes)
        {
            void* p = nullptr;
            int rc = workspace(tr_bytes + col_bytes, s, &p);
            if (rc)
                return rc;
            ws = static_cast<uint8_t*>(p);
        }
        if (tr_in)
        {
            int rc = launch_transpose(data, ws, g.N, g.C, in_sp, 1, s);
            if (rc)
                return rc;
            x = ws;
        }
        if (as_gemm)
        {
            if (!pointwise)
            {
                int rc = launch_im2col_nxc(g, x, ws + tr_bytes, zp.data_zp, zp.data_t, s);
                if (rc)
                    return rc;
                x = ws + tr_bytes;
            }
            hipq_dot_desc_t dd;
            memset(&dd, 0, sizeof(dd));
            dd.a_t = g.data_t;
            dd.b_t = g.filter_t;
            dd.out_t = g.out_t;
            dd.M = M;
            dd.K = kred;
            dd.N = g.K;
            if (dot_mfma_eligible(dd))
            {
                const int32_t* wsum = reinterpret_cast<const int32_t*>(static_cast<const uint8_t*>(packed) + align_up(static_cast<size_t>(g.K * kred), 256));
                return launch_dot_mfma(dd, x, packed, wsum, zp, epi, out, s);
            }
        }
        const bool out_ncx = g.out_layout == HIPQ_LAYOUT_NCX && g.K > 1;
        // layers whose filter fits in LDS take the band kernel (HIPQ_NO_BAND=1 forces the generic one)
        const bool no_band = getenv("HIPQ_NO_BAND") != nullptr;
        // (a 1 x 1 filter over every pixel, 8-bit channels-last output in whole 16-byte rows: the data
        // is a row matrix and the tile kernels that load it straight into LDS are faster -- 64 -> 64
        // channels at 56 x 56, batch 128: 15.8 us against 23 us)
        const bool row_matrix = !out_ncx && g.taps() == 1 && g.st[1] == 1 && g.st[2] == 1 && g.pb[1] == 0 && g.pb[2] == 0 && g.out[1] == g.in[1] && g.out[2] == g.in[2] &&
                                (g.out_t == HIPQ_U8 || g.out_t == HIPQ_I8) && g.K % 16 == 0 && getenv("HIPQ_NO_DMA") == nullptr && getenv("HIPQ_NO_PIPE") == nullptr;
        if (!no_band && !row_matrix && conv_band_eligible(g, out_ncx))
            return launch_conv_band(g, x, packed, zp, epi, out, out_ncx, s);
        return launch_conv_mfma(g, x, packed, zp, epi, out, out_ncx, s);
    }

    static int fused_epilogue(const hipq_fused_desc_t* f,
                              int out_t,
                              int64_t channels,
                              const int32_t* bias,
                              const void* sum_in,
                              const float* scale,
                              const float* sum_scale,
                              Epilogue* e)
    {
        HIPQ_REQUIRE(f, "fused descriptor is null");
        HIPQ_REQUIRE(scale, "scale is null");
        HIPQ_REQUIRE(f->scale_count == 1 || f->scale_count == channels,
                     "scale_count %lld is neither 1 nor the channel count %lld",
                     (long long)f->scale_count,
                     (long long)channels);
        HIPQ_REQUIRE(!f->has_bias || bias, "has_bias set but bias is null");
        HIPQ_REQUIRE(!f->has_sum || (sum_in && sum_scale), "has_sum set but sum_in / sum_scale is null");
        if (f->has_sum && !is_quant8(f->sum_t))
            return fail(HIPQ_ERR_UNSUPPORTED, "sum input must be u8 or i8");
        memset(e, 0, sizeof(*e));
        e->mode = EPI_FUSED;
        e->out_t = out_t;
        e->bias = f->has_bias ? bias : nullptr;
        e->scale = scale;
        e->per_channel = f->scale_count > 1;
        e->sum_in = f->has_sum ? sum_in : nullptr;
        e->sum_scale = f->has_sum ? sum_scale : nullptr;
        e->sum_t = f->sum_t;
        e->relu = f->with_relu;
        return HIPQ_OK;
    }

    static int dot_pack(const hipq_dot_desc_t& d, const void* b, void* packed, bool with_fragments, hipStream_t s);

    // Layout of a packed dot operand: [N][K] weights (only when the caller's are [K][N]), the column
    // sums, and -- for products the weight-streaming kernels take -- the weights once more in MFMA
    // fragment order.  Each part starts on a 256-byte boundary.
    static size_t dot_blob_weights(const hipq_dot_desc_t& d) { return d.b_layout == HIPQ_B_KN ? align_up(static_cast<size_t>(d.N * d.K), 256) : 0; }
    static size_t dot_blob_sums(const hipq_dot_desc_t& d) { return align_up(static_cast<size_t>(d.N) * sizeof(int32_t), 256); }

    // weights [N,K] + column sums for the MFMA dot, either prepacked or built in the workspace
    // (built on the fly there is no fragment-ordered copy: making one costs more than it saves a call)
    static int dot_operands(const hipq_dot_desc_t& d, const void* b, const void* packed, const void** w, const int32_t** wsum, const void** wfrag, hipStream_t s)
    {
        const size_t wbytes = dot_blob_weights(d);
        const uint8_t* blob = static_cast<const uint8_t*>(packed);
        *wfrag = nullptr;
        if (!blob)
        {
            uint8_t* ws = nullptr;
            int rc = workspace(wbytes + dot_blob_sums(d), s, reinterpret_cast<void**>(&ws));
            if (rc)
                return rc;
            rc = dot_pack(d, b, ws, false, s);
            if (rc)
                return rc;
            blob = ws;
        }
        else if (dot_fragments_eligible(d))
            *wfrag = blob + wbytes + dot_blob_sums(d);
        *w = d.b_layout == HIPQ_B_KN ? static_cast<const void*>(blob) : b;
        *wsum = reinterpret_cast<const int32_t*>(blob + wbytes);
        return HIPQ_OK;
    }

    static int run_dot(const hipq_dot_desc_t& d,
                       const void* a,
                       const void* b,
                       const void* packed,
                       const ZeroPoints& zp,
                       const Epilogue& epi,
                       void* out,
                       hipStream_t s)
    {
        if (d.M == 0 || d.N == 0)
            return HIPQ_OK;
        HIPQ_REQUIRE(out && (d.K == 0 || (a && b)), "null tensor pointer");
        if (!dot_mfma_eligible(d) || (reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15) ||
            (reinterpret_cast<uintptr_t>(out) & 15))
            return launch_dot_direct(d, a, b, zp, epi, out, s);
        const void* w = nullptr;
        const void* wfrag = nullptr;
        const int32_t* wsum = nullptr;
        int rc = dot_operands(d, b, packed, &w, &wsum, &wfrag, s);
        if (rc)
            return rc;
        return launch_dot_mfma(d, a, w, wsum, zp, epi, out, s, wfrag);
    }

    static int dot_pack(const hipq_dot_desc_t& d, const void* b, void* packed, bool with_fragments, hipStream_t s)
    {
        uint8_t* blob = static_cast<uint8_t*>(packed);
        const void* w = b;
        const size_t wbytes = dot_blob_weights(d);
        if (d.b_layout == HIPQ_B_KN)
        {
            int rc = launch_transpose(b, blob, 1, d.K, d.N, 1, s); // [K][N] -> [N][K]
            if (rc)
                return rc;
            w = blob;
        }
        int rc = launch_row_sums_i8(w, d.N, d.K, reinterpret_cast<int32_t*>(blob + wbytes), s);
        if (rc || !with_fragments || !dot_fragments_eligible(d))
            return rc;
        return launch_pack_dot_fragments(w, d.N, d.K, blob + wbytes + dot_blob_sums(d), s);
    }
}

using namespace hipq;

extern "C" {

int hipq_conv_infer_output(hipq_conv_desc_t* d)
{
    HIPQ_REQUIRE(d, "descriptor is null");
    HIPQ_REQUIRE(d->n_spatial >= 1 && d->n_spatial <= HIPQ_MAX_SPATIAL, "n_spatial %d out of range", d->n_spatial);
    for (int i = 0; i < d->n_spatial; ++i)
    {
        HIPQ_REQUIRE(d->in_sp[i] >= 1 && d->f_sp[i] >= 1 && d->stride[i] >= 1 && d->dilation[i] >= 1 && d->data_dilation[i] >= 1,
                     "non-positive extent, stride or dilation on spatial axis %d", i);
        int64_t in_eff = (d->in_sp[i] - 1) * d->data_dilation[i] + 1 + d->pad_below[i] + d->pad_above[i];
        int64_t f_eff = (d->f_sp[i] - 1) * d->dilation[i] + 1;
        HIPQ_REQUIRE(in_eff >= f_eff, "window larger than padded data on spatial axis %d", i);
        d->out_sp[i] = (in_eff - f_eff) / d->stride[i] + 1;
    }
    return HIPQ_OK;
}

int hipq_quantized_convolution(const hipq_conv_desc_t* desc,
                               const void* data,
                               const void* filter,
                               const void* packed_filter,
                               const float* data_scale,
                               const void* data_zp,
                               const float* filter_scale,
                               const void* filter_zp,
                               const float* out_scale,
                               const void* out_zp,
                               void* out,
                               void* stream)
{
    ConvGeom g;
    int rc = make_geom(desc, &g);
    if (rc)
        return rc;
    rc = check_conv_types(g, false);
    if (rc)
        return rc;
    HIPQ_REQUIRE(data && filter && out, "null tensor pointer");
    HIPQ_REQUIRE(data_scale && data_zp && filter_scale && filter_zp && out_scale && out_zp, "null scale or zero point");
    Epilogue e;
    memset(&e, 0, sizeof(e));
    e.mode = EPI_INTERP;
    e.out_t = g.out_t;
    e.s_data = data_scale;
    e.s_filter = filter_scale;
    e.s_out = out_scale;
    e.out_zp = out_zp;
    ZeroPoints zp{data_zp, filter_zp, g.data_t, g.filter_t};
    return run_conv(g, data, filter, packed_filter, zp, e, out, as_stream(stream));
}

int hipq_quantized_convolution_noalloc(const hipq_conv_desc_t* desc,
                                       const void* data,
                                       const void* filter,
                                       const void* packed_filter,
                                       const float* data_scale,
                                       const void* data_zp,
                                       const float* filter_scale,
                                       const void* filter_zp,
                                       const float* out_scale,
                                       const void* out_zp,
                                       void* out,
                                       void* stream)
{
    // same kernels, same choices; whatever scratch they need comes out of the fixed per-device array
    int rc = noalloc_begin();
    if (rc)
        return rc;
    rc = hipq_quantized_convolution(desc, data, filter, packed_filter, data_scale, data_zp, filter_scale, filter_zp, out_scale, out_zp, out, stream);
    noalloc_end();
    return rc;
}

int hipq_quantized_convolution_fused(const hipq_conv_desc_t* desc,
                                     const hipq_fused_desc_t* fused,
                                     const void* data,
                                     const void* filter,
                                     const void* packed_filter,
                                     const int32_t* bias,
                                     const void* sum_in,
                                     const float* scale,
                                     const float* sum_scale,
                                     void* out,
                                     void* stream)
{
    ConvGeom g;
    int rc = make_geom(desc, &g);
    if (rc)
        return rc;
    rc = check_conv_types(g, true);
    if (rc)
        return rc;
    HIPQ_REQUIRE(data && filter && out, "null tensor pointer");
    Epilogue e;
    rc = fused_epilogue(fused, g.out_t, g.K, bias, sum_in, scale, sum_scale, &e);
    if (rc)
        return rc;
    ZeroPoints zp{nullptr, nullptr, g.data_t, g.filter_t};
    return run_conv(g, data, filter, packed_filter, zp, e, out, as_stream(stream));
}

// MaxPool over the output of a fused convolution, as the pair of descriptors the two calls would take
static int conv_pool_pair(const hipq_conv_desc_t* desc, const hipq_fused_desc_t* fused, const hipq_pool_desc_t* pool, ConvGeom* g, PoolFuse* pf)
{
    int rc = make_geom(desc, g);
    if (rc)
        return rc;
    rc = check_conv_types(*g, true);
    if (rc)
        return rc;
    HIPQ_REQUIRE(fused && pool, "descriptor is null");
    if (g->in[0] != 1 || pool->op != HIPQ_POOL_MAX || pool->n_spatial != 2 || desc->n_spatial != 2 || pool->dtype != g->out_t || pool->layout != g->out_layout || pool->N != g->N ||
        pool->C != g->K || pool->in_sp[0] != g->out[1] || pool->in_sp[1] != g->out[2] || fused->has_sum)
        return fail(HIPQ_ERR_UNSUPPORTED, "not a 2-D MaxPool over this convolution's output");
    hipq_pool_desc_t pd = *pool;
    rc = hipq_pool_infer_output(&pd);
    if (rc)
        return rc;
    pf->wh = pool->window[0];
    pf->ww = pool->window[1];
    pf->sh = pool->stride[0];
    pf->sw = pool->stride[1];
    pf->pt = pool->pad_below[0];
    pf->pl = pool->pad_below[1];
    pf->out_h = pd.out_sp[0];
    pf->out_w = pd.out_sp[1];
    return HIPQ_OK;
}

int hipq_conv_max_pool_fusable(const hipq_conv_desc_t* desc, const hipq_fused_desc_t* fused, const hipq_pool_desc_t* pool)
{
    ConvGeom g;
    PoolFuse pf;
    if (!desc || !fused || !pool || conv_pool_pair(desc, fused, pool, &g, &pf) != HIPQ_OK)
        return 0;
    Epilogue e;
    memset(&e, 0, sizeof(e));
    e.mode = EPI_FUSED;
    e.out_t = g.out_t;
    ZeroPoints zp{nullptr, nullptr, g.data_t, g.filter_t};
    RowPack rp;
    return conv_rowpack_eligible(g, &rp) && conv_stem_eligible(g, e, zp, &pf) ? 1 : 0;
}

int hipq_quantized_convolution_fused_max_pool(const hipq_conv_desc_t* desc,
                                              const hipq_fused_desc_t* fused,
                                              const hipq_pool_desc_t* pool,
                                              const void* data,
                                              const void* packed_filter,
                                              const int32_t* bias,
                                              const float* scale,
                                              void* out,
                                              void* stream)
{
    ConvGeom g;
    PoolFuse pf;
    int rc = conv_pool_pair(desc, fused, pool, &g, &pf);
    if (rc)
        return rc;
    HIPQ_REQUIRE(data && packed_filter && out, "null tensor pointer");
    Epilogue e;
    rc = fused_epilogue(fused, g.out_t, g.K, bias, nullptr, scale, nullptr, &e);
    if (rc)
        return rc;
    ZeroPoints zp{nullptr, nullptr, g.data_t, g.filter_t};
    RowPack rp;
    if (!conv_rowpack_eligible(g, &rp) || !conv_stem_eligible(g, e, zp, &pf))
        return fail(HIPQ_ERR_UNSUPPORTED, "this convolution / MaxPool pair has no fused kernel (hipq_conv_max_pool_fusable is 0)");
    return launch_conv_stem(g, data, packed_filter, zp, e, &pf, out, as_stream(stream));
}

size_t hipq_dot_packed_bytes(const hipq_dot_desc_t* d)
{
    if (!d || !dot_mfma_eligible(*d))
        return 0;
    return dot_blob_weights(*d) + dot_blob_sums(*d) + (dot_fragments_eligible(*d) ? dot_fragment_bytes(*d) : 0);
}

int hipq_dot_pack(const hipq_dot_desc_t* d, const void* b, void* packed, void* stream)
{
    HIPQ_REQUIRE(d && b && packed, "null pointer");
    if (!dot_mfma_eligible(*d))
        return fail(HIPQ_ERR_UNSUPPORTED, "shape is not eligible for the MFMA path (hipq_dot_packed_bytes is 0)");
    return dot_pack(*d, b, packed, true, as_stream(stream));
}

int hipq_quantized_dot(const hipq_dot_desc_t* d,
                       const void* a,
                       const void* b,
                       const void* packed_b,
                       const float* a_scale,
                       const void* a_zp,
                       const float* b_scale,
                       const void* b_zp,
                       const float* out_scale,
                       const void* out_zp,
                       void* out,
                       void* stream)
{
    HIPQ_REQUIRE(d, "descriptor is null");
    HIPQ_REQUIRE(d->M >= 0 && d->N >= 0 && d->K >= 0, "negative extent");
    HIPQ_REQUIRE(d->b_layout == HIPQ_B_KN || d->b_layout == HIPQ_B_NK, "bad b_layout");
    if (!is_quant8(d->a_t) || !is_quant8(d->b_t) || (!is_quant8(d->out_t) && d->out_t != HIPQ_I32))
        return fail(HIPQ_ERR_UNSUPPORTED, "QuantizedDot takes u8/i8 operands and gives i8, u8 or i32");
    HIPQ_REQUIRE(a_scale && a_zp && b_scale && b_zp && out_scale && out_zp, "null scale or zero point");
    Epilogue e;
    memset(&e, 0, sizeof(e));
    e.mode = EPI_INTERP;
    e.out_t = d->out_t;
    e.s_data = a_scale;
    e.s_filter = b_scale;
    e.s_out = out_scale;
    e.out_zp = out_zp;
    ZeroPoints zp{a_zp, b_zp, d->a_t, d->b_t};
    return run_dot(*d, a, b, packed_b, zp, e, out, as_stream(stream));
}

int hipq_quantized_dot_bias(const hipq_dot_desc_t* d,
                            const hipq_fused_desc_t* fused,
                            const void* a,
                            const void* w,
                            const void* packed_w,
                            const int32_t* bias,
                            const float* scale,
                            void* out,
                            void* stream)
{
    HIPQ_REQUIRE(d, "descriptor is null");
    HIPQ_REQUIRE(d->M >= 0 && d->N >= 0 && d->K >= 0, "negative extent");
    HIPQ_REQUIRE(d->b_layout == HIPQ_B_KN || d->b_layout == HIPQ_B_NK, "bad b_layout");
    if (!is_quant8(d->a_t) || d->b_t != HIPQ_I8 || (!is_quant8(d->out_t) && d->out_t != HIPQ_F32))
        return fail(HIPQ_ERR_UNSUPPORTED, "QuantizedDotBias takes u8/i8 data, i8 weights and gives i8, u8 or f32");
    HIPQ_REQUIRE(fused && !fused->has_sum, "QuantizedDotBias has no sum input");
    Epilogue e;
    int rc = fused_epilogue(fused, d->out_t, d->N, bias, nullptr, scale, nullptr, &e);
    if (rc)
        return rc;
    ZeroPoints zp{nullptr, nullptr, d->a_t, d->b_t};
    return run_dot(*d, a, w, packed_w, zp, e, out, as_stream(stream));
}

int hipq_quantized_dot_bias_gelu_quantize(const hipq_dot_desc_t* d,
                                          const hipq_fused_desc_t* fused,
                                          const void* a,
                                          const void* w,
                                          const void* packed_w,
                                          const int32_t* bias,
                                          const float* scale,
                                          const hipq_quant_out_t* quant,
                                          void* stream)
{
    HIPQ_REQUIRE(d, "descriptor is null");
    HIPQ_REQUIRE(d->M >= 0 && d->N >= 0 && d->K >= 0, "negative extent");
    HIPQ_REQUIRE(d->b_layout == HIPQ_B_KN || d->b_layout == HIPQ_B_NK, "bad b_layout");
    if (!is_quant8(d->a_t) || d->b_t != HIPQ_I8 || d->out_t != HIPQ_F32)
        return fail(HIPQ_ERR_UNSUPPORTED, "QuantizedDotBias + Gelu + Quantize takes u8/i8 data, i8 weights and the f32 form of the product (out_t F32)");
    HIPQ_REQUIRE(fused && !fused->has_sum, "QuantizedDotBias has no sum input");
    HIPQ_REQUIRE(quant && quant->out && quant->scale, "quantized output: null pointer");
    HIPQ_REQUIRE(quant->quant_t == HIPQ_I8 || quant->quant_t == HIPQ_U8, "quantized output: i8 or u8");
    HIPQ_REQUIRE(quant->round_mode >= HIPQ_ROUND_NEAREST_TOWARD_INFINITY && quant->round_mode <= HIPQ_ROUND_DOWN, "quantized output: unknown round mode");
    if (d->M == 0 || d->N == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(d->K == 0 || (a && w), "null tensor pointer");
    {
        // workgroups write their output bytes while others still read rows of `a`
        const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), a1 = a0 + static_cast<size_t>(d->M * d->K);
        const uintptr_t o0 = reinterpret_cast<uintptr_t>(quant->out), o1 = o0 + static_cast<size_t>(d->M * d->N);
        HIPQ_REQUIRE(a1 <= o0 || o1 <= a0, "the quantized output must not overlap the input rows");
    }
    Epilogue e;
    int rc = fused_epilogue(fused, HIPQ_F32, d->N, bias, nullptr, scale, nullptr, &e);
    if (rc)
        return rc;
    hipStream_t s = as_stream(stream);
    // in the epilogue of the product, where the kernels that take it apply
    if (dot_mfma_eligible(*d) && d->M > 256 && (reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0 && (reinterpret_cast<uintptr_t>(quant->out) & 15) == 0)
    {
        const void* wn = nullptr;
        const void* wfrag = nullptr;
        const int32_t* wsum = nullptr;
        rc = dot_operands(*d, w, packed_w, &wn, &wsum, &wfrag, s);
        if (rc)
            return rc;
        Epilogue post = e;
        post.post_scale = quant->scale;
        post.post_zp = quant->zero_point;
        post.post_t = quant->quant_t;
        post.post_mode = quant->round_mode;
        ZeroPoints zp{nullptr, nullptr, d->a_t, d->b_t};
        rc = launch_rows_gelu_q8(a, d->a_t == HIPQ_U8, static_cast<const int8_t*>(wn), wsum, d->M, static_cast<int32_t>(d->N), static_cast<int32_t>(d->K), zp, post, quant->out, s);
        if (rc != HIPQ_ERR_UNSUPPORTED)
            return rc;
    }
    // otherwise the product into the workspace, then Gelu + Quantize from there (prepacked weights only:
    // weights packed on the fly live in the same workspace)
    if (!packed_w)
        return fail(HIPQ_ERR_UNSUPPORTED, "QuantizedDotBias + Gelu + Quantize outside the fused kernels needs prepacked weights (hipq_dot_pack)");
    float* product = nullptr;
    rc = workspace(static_cast<size_t>(d->M) * static_cast<size_t>(d->N) * sizeof(float), s, reinterpret_cast<void**>(&product));
    if (rc)
        return rc;
    ZeroPoints zp{nullptr, nullptr, d->a_t, d->b_t};
    rc = run_dot(*d, a, w, packed_w, zp, e, product, s);
    if (rc)
        return rc;
    return hipq_gelu_quantize_f32(product, nullptr, quant, d->M * d->N, stream);
}
}
