// fp32 glue of a transformer encoder between the quantized projections: Softmax, Erf, Gelu,
// LayerNorm.  All of them stream their tensors once through HBM; a row (the normalised axis) is
// owned by one wavefront and kept in registers when it has at most 2048 elements.
#include <cmath>

#include "hipq_common.h"
#include "hipq_quant_math.h"
#include "hipq_row_math.h"

namespace hipq
{
    namespace
    {
        typedef float f4 __attribute__((ext_vector_type(4)));

        // the optional quantized copy of an output: Quantize with one scale and zero point for the whole
        // tensor, computed from the f32 value as it is stored (same arithmetic as hipq_quantize)
        struct QuantOut
        {
            void* out; // null: none
            const float* scale;
            const void* zero_point;
            int32_t quant_t, mode;
        };
        __device__ __forceinline__ uint32_t quant4(const QuantOut& q, float s, int32_t zp, f4 v)
        {
            // round half to even (uniform): the Quantize kernels' own four-at-a-time arithmetic
            if (q.mode == HIPQ_ROUND_NEAREST_TOWARD_EVEN)
                return q.quant_t == HIPQ_U8 ? quantize4<uint8_t, true>(v, s, static_cast<float>(zp), q.mode) : quantize4<int8_t, true>(v, s, static_cast<float>(zp), q.mode);
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e)
            {
                const uint32_t b = q.quant_t == HIPQ_U8 ? static_cast<uint32_t>(quantize_one<float, uint8_t>(v[e], s, static_cast<uint8_t>(zp), q.mode))
                                                        : static_cast<uint32_t>(static_cast<uint8_t>(quantize_one<float, int8_t>(v[e], s, static_cast<int8_t>(zp), q.mode)));
                w |= b << (8 * e);
            }
            return w;
        }
        __device__ __forceinline__ void quant1(const QuantOut& q, float s, int32_t zp, float v, int64_t i)
        {
            if (q.quant_t == HIPQ_U8)
                static_cast<uint8_t*>(q.out)[i] = quantize_one<float, uint8_t>(v, s, static_cast<uint8_t>(zp), q.mode);
            else
                static_cast<int8_t*>(q.out)[i] = quantize_one<float, int8_t>(v, s, static_cast<int8_t>(zp), q.mode);
        }

        constexpr int kRowVecs = 8; // float4 pieces of a row a lane keeps: rows up to 64 * 4 * 8 = 2048 elements

        // out = exp(x - max(x)) / sum(exp(x - max(x))) along contiguous rows
        // (src/ngraph/runtime/reference/softmax.hpp:31-57); one wavefront a row.
        template <bool CACHED>
        __global__ __launch_bounds__(256) void softmax_rows_kernel(const float* __restrict__ in, const float* __restrict__ factor, float* __restrict__ out, int64_t rows, int32_t cols)
        {
            // factor (may be null): the input is Multiply(x, factor) -- the product is rounded to f32 as the
            // Multiply op would round it
            const bool scaled = factor != nullptr;
            const float c = scaled ? *factor : 1.0f;
            const int lane = threadIdx.x & 63;
            const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
            if (row >= rows)
                return;
            const float* x = in + row * cols;
            float* y = out + row * cols;
            if (CACHED) // cols % 4 == 0, 16-byte aligned rows, cols <= 2048
            {
                const int vecs = cols >> 2;
                f4 v[kRowVecs];
                float m = -INFINITY;
#pragma unroll
                for (int i = 0; i < kRowVecs; ++i)
                {
                    const int j = i * 64 + lane;
                    if (j < vecs)
                    {
                        v[i] = reinterpret_cast<const f4*>(x)[j];
                        if (scaled)
                            v[i] = f4{__fmul_rn(v[i][0], c), __fmul_rn(v[i][1], c), __fmul_rn(v[i][2], c), __fmul_rn(v[i][3], c)};
                        m = fmaxf(fmaxf(fmaxf(m, v[i][0]), fmaxf(v[i][1], v[i][2])), v[i][3]);
                    }
                }
                m = wave_max(m);
                float s = 0.0f;
#pragma unroll
                for (int i = 0; i < kRowVecs; ++i)
                    if (i * 64 + lane < vecs)
                    {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                        {
                            v[i][e] = expf(v[i][e] - m);
                            s += v[i][e];
                        }
                    }
                s = wave_sum(s);
#pragma unroll
                for (int i = 0; i < kRowVecs; ++i)
                {
                    const int j = i * 64 + lane;
                    if (j < vecs)
                        reinterpret_cast<f4*>(y)[j] = f4{v[i][0] / s, v[i][1] / s, v[i][2] / s, v[i][3] / s};
                }
            }
            else
            {
                auto at = [&](int j) { return scaled ? __fmul_rn(x[j], c) : x[j]; };
                float m = -INFINITY;
                for (int j = lane; j < cols; j += 64)
                    m = fmaxf(m, at(j));
                m = wave_max(m);
                float s = 0.0f;
                for (int j = lane; j < cols; j += 64)
                    s += expf(at(j) - m);
                s = wave_sum(s);
                for (int j = lane; j < cols; j += 64)
                    y[j] = expf(at(j) - m) / s;
            }
        }

        // short rows (at most W float4 pieces, W = 32, 16 or 8 lanes): 64 / W rows a wavefront, one
        // piece a lane, so that every lane has work (an attention row of 128 is 32 pieces)
        template <int W>
        __global__ __launch_bounds__(256) void softmax_short_rows_kernel(const float* __restrict__ in, const float* __restrict__ factor, float* __restrict__ out, int64_t rows, int32_t cols)
        {
            const bool scaled = factor != nullptr;
            const float c = scaled ? *factor : 1.0f;
            constexpr int RPW = 64 / W;
            const int lane = threadIdx.x & 63;
            const int sub = lane & (W - 1);
            const int64_t row = (static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6)) * RPW + lane / W;
            const int vecs = cols >> 2;
            const bool live = row < rows && sub < vecs;
            f4 v = f4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
            if (live)
                v = reinterpret_cast<const f4*>(in + row * cols)[sub];
            v = softmax_piece<W>(v, live, scaled, c);
            if (live)
                reinterpret_cast<f4*>(out + row * cols)[sub] = v;
        }

        // the same over a strided axis: the tensor is [outer][axis][inner], one lane a column (o, i)
        __global__ __launch_bounds__(256) void softmax_strided_kernel(const float* __restrict__ in, const float* __restrict__ factor, float* __restrict__ out, int64_t outer, int32_t axis, int64_t inner)
        {
            const bool scaled = factor != nullptr;
            const float c = scaled ? *factor : 1.0f;
            const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
            if (t >= outer * inner)
                return;
            const int64_t o = t / inner, i = t - o * inner;
            const float* x = in + o * axis * inner + i;
            float* y = out + o * axis * inner + i;
            auto at = [&](int a) { return scaled ? __fmul_rn(x[a * inner], c) : x[a * inner]; };
            float m = -INFINITY;
            for (int a = 0; a < axis; ++a)
                m = fmaxf(m, at(a));
            float s = 0.0f;
            for (int a = 0; a < axis; ++a)
                s += expf(at(a) - m);
            for (int a = 0; a < axis; ++a)
                y[a * inner] = expf(at(a) - m) / s;
        }

        template <bool GELU>
        __global__ __launch_bounds__(256) void erf_kernel(const float* __restrict__ in, float* __restrict__ out, QuantOut q, int64_t count, int32_t vec_ok)
        {
            // out may be null when only the quantized copy is wanted
            const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
            const float qs = q.out ? *q.scale : 1.0f;
            const int32_t qz = q.out ? load_zp(q.zero_point, q.quant_t) : 0;
            if (vec_ok)
            {
                if (t * 4 >= count)
                    return;
                const f4 v = reinterpret_cast<const f4*>(in)[t];
                f4 r;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    r[e] = GELU ? gelu1(v[e]) : erff(v[e]);
                if (out)
                    reinterpret_cast<f4*>(out)[t] = r;
                if (q.out)
                    static_cast<uint32_t*>(q.out)[t] = quant4(q, qs, qz, r);
            }
            else if (t < count)
            {
                const float r = GELU ? gelu1(in[t]) : erff(in[t]);
                if (out)
                    out[t] = r;
                if (q.out)
                    quant1(q, qs, qz, r, t);
            }
        }

        // LayerNorm over the trailing `cols` elements of every row, as the reference decomposes it
        // (src/ngraph/op/layer_norm.cpp:96-139 with builder::mean / builder::variance,
        // src/ngraph/builder/reduce_ops.cpp:68-124): mean = sum(x) / n, var = sum((x - mean)^2) / n,
        // out = (x - mean) / sqrt(var + eps) * scale + bias.  One wavefront a row.
        template <bool CACHED>
        __global__ __launch_bounds__(256) void layer_norm_kernel(const float* __restrict__ in, const float* __restrict__ addend, const float* __restrict__ scale,
                                                                 const float* __restrict__ bias, float* __restrict__ out, QuantOut qo, float* __restrict__ mean_out,
                                                                 float* __restrict__ var_out, int64_t rows, int32_t cols, float eps)
        {
            // addend (may be null): the input is Add(in, addend), the sum rounded to f32 as the Add op rounds it;
            // qo.out (may be null): Quantize of the result beside it
            const int lane = threadIdx.x & 63;
            const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
            if (row >= rows)
                return;
            const float* x = in + row * cols;
            const float* x2 = addend ? addend + row * cols : nullptr;
            float* y = out + row * cols;
            const float n = static_cast<float>(cols);
            const float qs = qo.out ? *qo.scale : 1.0f;
            const int32_t qz = qo.out ? load_zp(qo.zero_point, qo.quant_t) : 0;
            if (CACHED)
            {
                const int vecs = cols >> 2;
                f4 v[kRowVecs];
                float s = 0.0f;
#pragma unroll
                for (int i = 0; i < kRowVecs; ++i)
                    if (i * 64 + lane < vecs)
                    {
                        v[i] = reinterpret_cast<const f4*>(x)[i * 64 + lane];
                        if (x2)
                        {
                            const f4 w = reinterpret_cast<const f4*>(x2)[i * 64 + lane];
                            v[i] = f4{__fadd_rn(v[i][0], w[0]), __fadd_rn(v[i][1], w[1]), __fadd_rn(v[i][2], w[2]), __fadd_rn(v[i][3], w[3])};
                        }
                        s += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);
                    }
                const float mean = __fdiv_rn(wave_sum(s), n);
                float q = 0.0f;
#pragma unroll
                for (int i = 0; i < kRowVecs; ++i)
                    if (i * 64 + lane < vecs)
                    {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                        {
                            v[i][e] = v[i][e] - mean;
                            q = fmaf(v[i][e], v[i][e], q);
                        }
                    }
                const float var = __fdiv_rn(wave_sum(q), n);
                const float sd = sqrtf(var + eps);
                // one division a row: the elements divide through its reciprocal, which gives the division's
                // own result for every normal quotient (a row whose deviation is zero, infinite or out of
                // the reciprocal's range keeps the division)
                const float rsd = __fdiv_rn(1.0f, sd);
                const bool by_reciprocal = sd > 1e-30f && sd < 1e30f; // uniform
#pragma unroll
                for (int i = 0; i < kRowVecs; ++i)
                {
                    const int j = i * 64 + lane;
                    if (j < vecs)
                    {
                        f4 r;
                        const f4 sc = scale ? reinterpret_cast<const f4*>(scale)[j] : f4{1.0f, 1.0f, 1.0f, 1.0f};
                        const f4 bi = scale ? reinterpret_cast<const f4*>(bias)[j] : f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                        {
                            const float nv = by_reciprocal ? div_by_reciprocal(v[i][e], sd, rsd) : __fdiv_rn(v[i][e], sd);
                            r[e] = scale ? __fadd_rn(__fmul_rn(nv, sc[e]), bi[e]) : nv;
                        }
                        reinterpret_cast<f4*>(y)[j] = r;
                        if (qo.out)
                            static_cast<uint32_t*>(qo.out)[(row * cols >> 2) + j] = quant4(qo, qs, qz, r);
                    }
                }
                if (lane == 0)
                {
                    if (mean_out)
                        mean_out[row] = mean;
                    if (var_out)
                        var_out[row] = var;
                }
            }
            else
            {
                auto at = [&](int j) { return x2 ? __fadd_rn(x[j], x2[j]) : x[j]; };
                float s = 0.0f;
                for (int j = lane; j < cols; j += 64)
                    s += at(j);
                const float mean = __fdiv_rn(wave_sum(s), n);
                float q = 0.0f;
                for (int j = lane; j < cols; j += 64)
                {
                    const float d = at(j) - mean;
                    q = fmaf(d, d, q);
                }
                const float var = __fdiv_rn(wave_sum(q), n);
                const float sd = sqrtf(var + eps);
                for (int j = lane; j < cols; j += 64)
                {
                    const float nv = __fdiv_rn(at(j) - mean, sd);
                    const float r = scale ? __fadd_rn(__fmul_rn(nv, scale[j]), bias[j]) : nv;
                    y[j] = r;
                    if (qo.out)
                        quant1(qo, qs, qz, r, row * cols + j);
                }
                if (lane == 0)
                {
                    if (mean_out)
                        mean_out[row] = mean;
                    if (var_out)
                        var_out[row] = var;
                }
            }
        }

        bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
    }
}

using namespace hipq;

static int launch_softmax(const float* in, const float* factor, float* out, int64_t outer, int64_t axis, int64_t inner, void* stream)
{
    HIPQ_REQUIRE(outer >= 0 && axis >= 0 && inner >= 0, "negative extent");
    if (outer == 0 || axis == 0 || inner == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && out, "null pointer");
    HIPQ_REQUIRE(axis < (1ll << 31) && outer * inner < (1ll << 40), "tensor too large for one launch");
    hipStream_t s = as_stream(stream);
    if (inner == 1)
    {
        const bool cached = axis % 4 == 0 && axis <= 64 * 4 * kRowVecs && aligned16(in) && aligned16(out);
        if (cached && axis <= 128)
        {
            const int w = axis > 64 ? 32 : (axis > 32 ? 16 : 8);
            const int64_t rows_per_block = 4 * (64 / w);
            const unsigned blocks = static_cast<unsigned>((outer + rows_per_block - 1) / rows_per_block);
            if (w == 32)
                softmax_short_rows_kernel<32><<<blocks, 256, 0, s>>>(in, factor, out, outer, static_cast<int32_t>(axis));
            else if (w == 16)
                softmax_short_rows_kernel<16><<<blocks, 256, 0, s>>>(in, factor, out, outer, static_cast<int32_t>(axis));
            else
                softmax_short_rows_kernel<8><<<blocks, 256, 0, s>>>(in, factor, out, outer, static_cast<int32_t>(axis));
            return check_launch("softmax_rows");
        }
        const unsigned grid = static_cast<unsigned>((outer + 3) / 4);
        if (cached)
            softmax_rows_kernel<true><<<grid, 256, 0, s>>>(in, factor, out, outer, static_cast<int32_t>(axis));
        else
            softmax_rows_kernel<false><<<grid, 256, 0, s>>>(in, factor, out, outer, static_cast<int32_t>(axis));
        return check_launch("softmax_rows");
    }
    softmax_strided_kernel<<<static_cast<unsigned>((outer * inner + 255) / 256), 256, 0, s>>>(in, factor, out, outer, static_cast<int32_t>(axis), inner);
    return check_launch("softmax_strided");
}

int hipq_softmax_f32(const float* in, float* out, int64_t outer, int64_t axis, int64_t inner, void* stream)
{
    return launch_softmax(in, nullptr, out, outer, axis, inner, stream);
}

int hipq_softmax_scaled_f32(const float* in, const float* factor, float* out, int64_t outer, int64_t axis, int64_t inner, void* stream)
{
    HIPQ_REQUIRE(factor, "null factor");
    return launch_softmax(in, factor, out, outer, axis, inner, stream);
}

// the caller's description of a quantized side output -> the kernels' (null: none)
static int quant_out(const hipq_quant_out_t* q, QuantOut* r)
{
    *r = QuantOut{nullptr, nullptr, nullptr, HIPQ_I8, HIPQ_ROUND_NEAREST_TOWARD_EVEN};
    if (!q)
        return HIPQ_OK;
    HIPQ_REQUIRE(q->out && q->scale, "quantized output: null pointer");
    HIPQ_REQUIRE(q->quant_t == HIPQ_I8 || q->quant_t == HIPQ_U8, "quantized output: i8 or u8");
    HIPQ_REQUIRE(q->round_mode >= HIPQ_ROUND_NEAREST_TOWARD_INFINITY && q->round_mode <= HIPQ_ROUND_DOWN, "quantized output: unknown round mode");
    *r = QuantOut{q->out, q->scale, q->zero_point, q->quant_t, q->round_mode};
    return HIPQ_OK;
}

static int launch_erf(const float* in, float* out, const hipq_quant_out_t* q, int64_t count, void* stream, bool gelu)
{
    HIPQ_REQUIRE(count >= 0, "negative count");
    if (count == 0)
        return HIPQ_OK;
    QuantOut qo;
    if (const int rc = quant_out(q, &qo))
        return rc;
    HIPQ_REQUIRE(in && (out || qo.out), "null pointer");
    const bool vec = count % 4 == 0 && aligned16(in) && (!out || aligned16(out)) && (!qo.out || (reinterpret_cast<uintptr_t>(qo.out) & 3) == 0);
    const int64_t lanes = vec ? count / 4 : count;
    HIPQ_REQUIRE((lanes + 255) / 256 < (1ll << 31), "tensor too large for one launch");
    const unsigned grid = static_cast<unsigned>((lanes + 255) / 256);
    if (gelu)
        erf_kernel<true><<<grid, 256, 0, as_stream(stream)>>>(in, out, qo, count, vec ? 1 : 0);
    else
        erf_kernel<false><<<grid, 256, 0, as_stream(stream)>>>(in, out, qo, count, vec ? 1 : 0);
    return check_launch(gelu ? "gelu_vec" : "erf_vec");
}

int hipq_erf_f32(const float* in, float* out, int64_t count, void* stream)
{
    return launch_erf(in, out, nullptr, count, stream, false);
}

int hipq_gelu_f32(const float* in, float* out, int64_t count, void* stream)
{
    return launch_erf(in, out, nullptr, count, stream, true);
}

int hipq_gelu_quantize_f32(const float* in, float* out, const hipq_quant_out_t* q, int64_t count, void* stream)
{
    HIPQ_REQUIRE(q, "null quantized output");
    return launch_erf(in, out, q, count, stream, true);
}

static int launch_layer_norm(const float* in, const float* addend, const float* scale, const float* bias, float* out, const hipq_quant_out_t* q, float* mean, float* var,
                             int64_t rows, int64_t cols, double epsilon, void* stream)
{
    HIPQ_REQUIRE(rows >= 0 && cols >= 0, "negative extent");
    if (rows == 0 || cols == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && out, "null pointer");
    HIPQ_REQUIRE((scale == nullptr) == (bias == nullptr), "scale and bias come together");
    HIPQ_REQUIRE(cols < (1ll << 31) && (rows + 3) / 4 < (1ll << 31), "tensor too large for one launch");
    QuantOut qo;
    if (const int rc = quant_out(q, &qo))
        return rc;
    const bool cached = cols % 4 == 0 && cols <= 64 * 4 * kRowVecs && aligned16(in) && aligned16(out) && (!scale || (aligned16(scale) && aligned16(bias))) &&
                        (!addend || aligned16(addend)) && (!qo.out || (reinterpret_cast<uintptr_t>(qo.out) & 3) == 0);
    const unsigned grid = static_cast<unsigned>((rows + 3) / 4);
    hipStream_t s = as_stream(stream);
    if (cached)
        layer_norm_kernel<true><<<grid, 256, 0, s>>>(in, addend, scale, bias, out, qo, mean, var, rows, static_cast<int32_t>(cols), static_cast<float>(epsilon));
    else
        layer_norm_kernel<false><<<grid, 256, 0, s>>>(in, addend, scale, bias, out, qo, mean, var, rows, static_cast<int32_t>(cols), static_cast<float>(epsilon));
    return check_launch("layer_norm_rows");
}

int hipq_layer_norm_f32(const float* in, const float* scale, const float* bias, float* out, float* mean, float* var, int64_t rows, int64_t cols, double epsilon, void* stream)
{
    return launch_layer_norm(in, nullptr, scale, bias, out, nullptr, mean, var, rows, cols, epsilon, stream);
}

int hipq_add_layer_norm_f32(const float* a, const float* b, const float* scale, const float* bias, float* out, const hipq_quant_out_t* q, int64_t rows, int64_t cols, double epsilon,
                            void* stream)
{
    return launch_layer_norm(a, b, scale, bias, out, q, nullptr, nullptr, rows, cols, epsilon, stream);
}
