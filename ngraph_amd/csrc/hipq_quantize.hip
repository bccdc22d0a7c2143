// Quantize / Dequantize kernels (HBM-bound elementwise work).
//
// Arithmetic follows src/ngraph/runtime/reference/quantize.hpp:29-117 and dequantize.hpp:31-53 of
// the nGraph tree: true IEEE division by the scale, the reference's floor/ceil rounding formulas,
// zero point added in REAL, clamp in REAL, then the cast.
//
// Two kernel families:
//   *_vec4    f32 <-> {i8,u8}, scale laid along one run of adjacent axes (or scalar) and the
//             innermost non-axis extent a multiple of 4.  Each lane moves groups of 4 elements:
//             one 16-byte load/store on the f32 side, one 4-byte store/load on the quantized side,
//             lane-contiguous, so a wavefront touches 1 KiB + 256 B of consecutive memory per step.
//   *_generic every other case (f64, i32, ragged inner extent, scattered axes): one element per
//             lane, coordinates recovered with 64-bit div/mod.
#include "hipq_common.h"
#include "hipq_index_div.h"
#include "hipq_quant_math.h"

namespace hipq
{
    struct DimInfo
    {
        int32_t rank;
        uint32_t axes_mask;
        int64_t shape[HIPQ_MAX_RANK];
    };

    __device__ __forceinline__ int64_t project_index(const DimInfo& d, int64_t i)
    {
        int64_t coord[HIPQ_MAX_RANK];
        for (int a = d.rank - 1; a >= 0; --a)
        {
            coord[a] = i % d.shape[a];
            i /= d.shape[a];
        }
        int64_t j = 0;
        for (int a = 0; a < d.rank; ++a)
            if (d.axes_mask & (1u << a))
                j = j * d.shape[a] + coord[a];
        return j;
    }

    template <typename REAL, typename QUANT>
    __global__ __launch_bounds__(256) void quantize_generic_kernel(const REAL* __restrict__ in,
                                                                   const REAL* __restrict__ scale,
                                                                   const QUANT* __restrict__ zp,
                                                                   QUANT* __restrict__ out,
                                                                   int64_t count,
                                                                   DimInfo dims,
                                                                   int mode)
    {
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < count; i += stride)
        {
            int64_t j = dims.axes_mask ? project_index(dims, i) : 0;
            out[i] = quantize_one<REAL, QUANT>(in[i], scale[j], zp[j], mode);
        }
    }

    template <typename QUANT, typename REAL>
    __global__ __launch_bounds__(256) void dequantize_generic_kernel(const QUANT* __restrict__ in,
                                                                     const REAL* __restrict__ scale,
                                                                     const QUANT* __restrict__ zp,
                                                                     REAL* __restrict__ out,
                                                                     int64_t count,
                                                                     DimInfo dims)
    {
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < count; i += stride)
        {
            int64_t j = dims.axes_mask ? project_index(dims, i) : 0;
            // integer subtract after promotion; int32 wraps (dequantize.hpp:46-50)
            int32_t diff = static_cast<int32_t>(static_cast<uint32_t>(static_cast<int32_t>(in[i])) -
                                                static_cast<uint32_t>(static_cast<int32_t>(zp[j])));
            out[i] = static_cast<REAL>(diff) * scale[j];
        }
    }

    // ---- vectorised f32 <-> 8-bit path ----------------------------------------------------------
    // The tensor is viewed as [outer, A, inner] with the scale index = (i / inner) % A
    // (A == 1: scalar scale).  groups = count / 4; group g covers elements 4g .. 4g+3.
    struct RunView
    {
        IndexDiv div_inner4; // divides a group index by inner/4
        IndexDiv div_a;
        uint32_t a;         // extent of the scale table
    };

    __device__ __forceinline__ uint32_t run_index(const RunView& v, uint32_t group)
    {
        if (v.a == 1)
            return 0;
        uint32_t row = fastdiv(group, v.div_inner4);
        uint32_t q = fastdiv(row, v.div_a);
        return row - q * v.a;
    }

    // Groups a lane handles per launch, one wavefront-contiguous step of 256 groups apart (measured
    // on f32[64,1024,1024]: 3 is best for Quantize, 2 for Dequantize).
    constexpr int kQuantUnroll = 3;
    constexpr int kDequantUnroll = 2;

    // ROW_UNIFORM: inner/4 is a multiple of the 256 groups one step of a workgroup covers (or the
    // scale is a scalar), so a step lies inside one row of the scale table and its index comes from
    // the block index alone: scale and zero point arrive through the scalar unit instead of two
    // vector loads and two 64-bit multiplies per lane.
    template <bool ROW_UNIFORM>
    __device__ __forceinline__ uint32_t step_run_index(const RunView& v, uint32_t first_group_of_step, uint32_t g)
    {
        return run_index(v, ROW_UNIFORM ? first_group_of_step : g);
    }
    template <typename QUANT, bool RNE, bool ROW_UNIFORM>
    __global__ __launch_bounds__(256) void quantize_vec4_kernel(const f32x4* __restrict__ in,
                                                                const float* __restrict__ scale,
                                                                const QUANT* __restrict__ zp,
                                                                uint32_t* __restrict__ out,
                                                                uint32_t groups,
                                                                RunView view,
                                                                int mode)
    {
        constexpr int kUnroll = kQuantUnroll;
        uint32_t first = blockIdx.x * (256u * kUnroll);
        uint32_t base = first + threadIdx.x;
        f32x4 x[kUnroll];
        float s[kUnroll];
        float z[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            uint32_t g = base + u * 256u;
            if (g < groups)
            {
                x[u] = __builtin_nontemporal_load(&in[g]);
                uint32_t j = step_run_index<ROW_UNIFORM>(view, first + u * 256u, g);
                s[u] = scale[j];
                z[u] = static_cast<float>(zp[j]);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            uint32_t g = base + u * 256u;
            if (g < groups)
                __builtin_nontemporal_store(quantize4<QUANT, RNE>(x[u], s[u], z[u], mode), &out[g]);
        }
    }

    // The quantized side is read with ordinary loads (4 bytes a lane: streaming hints on so narrow a
    // load cost a sixth of the rate), the f32 side written with streaming stores.
    template <typename QUANT, bool ROW_UNIFORM>
    __global__ __launch_bounds__(256) void dequantize_vec4_kernel(const uint32_t* __restrict__ in,
                                                                  const float* __restrict__ scale,
                                                                  const QUANT* __restrict__ zp,
                                                                  f32x4* __restrict__ out,
                                                                  uint32_t groups,
                                                                  RunView view)
    {
        constexpr int kUnroll = kDequantUnroll;
        uint32_t first = blockIdx.x * (256u * kUnroll);
        uint32_t base = first + threadIdx.x;
        uint32_t q[kUnroll];
        float s[kUnroll];
        int32_t z[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            uint32_t g = base + u * 256u;
            if (g < groups)
            {
                q[u] = in[g];
                uint32_t j = step_run_index<ROW_UNIFORM>(view, first + u * 256u, g);
                s[u] = scale[j];
                z[u] = static_cast<int32_t>(zp[j]);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            uint32_t g = base + u * 256u;
            if (g < groups)
            {
                float r[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    int32_t v = static_cast<int32_t>(static_cast<QUANT>((q[u] >> (8 * e)) & 0xFFu));
                    r[e] = __fmul_rn(static_cast<float>(v - z[u]), s[u]);
                }
                f32x4 o = {r[0], r[1], r[2], r[3]};
                __builtin_nontemporal_store(o, &out[g]);
            }
        }
    }

    // ---- host side -------------------------------------------------------------------------------
    struct Canon
    {
        int64_t count;
        bool single_run; // scalar, or one run of adjacent axes
        int64_t outer, a, inner;
    };

    static Canon canonicalise(const hipq_quant_desc_t& d)
    {
        Canon c;
        c.count = 1;
        for (int i = 0; i < d.rank; ++i)
            c.count *= d.shape[i];
        c.outer = c.a = c.inner = 1;
        // 0 = before the run, 1 = in the run, 2 = after the run
        int state = 0;
        c.single_run = true;
        for (int i = 0; i < d.rank; ++i)
        {
            if (d.shape[i] == 1)
                continue;
            bool on_axis = (d.axes_mask >> i) & 1u;
            if (on_axis)
            {
                if (state == 2)
                    c.single_run = false;
                state = 1;
                c.a *= d.shape[i];
            }
            else if (state == 0)
                c.outer *= d.shape[i];
            else
            {
                state = 2;
                c.inner *= d.shape[i];
            }
        }
        return c;
    }

    static int check_desc(const hipq_quant_desc_t* d)
    {
        HIPQ_REQUIRE(d, "descriptor is null");
        HIPQ_REQUIRE(d->rank >= 0 && d->rank <= HIPQ_MAX_RANK, "rank %d out of range", d->rank);
        for (int i = 0; i < d->rank; ++i)
            HIPQ_REQUIRE(d->shape[i] >= 0, "negative extent");
        HIPQ_REQUIRE((d->axes_mask >> d->rank) == 0, "axes beyond rank");
        if (d->real_t != HIPQ_F32 && d->real_t != HIPQ_F64)
            return fail(HIPQ_ERR_UNSUPPORTED, "real type must be f32 or f64");
        if (d->quant_t != HIPQ_U8 && d->quant_t != HIPQ_I8 && d->quant_t != HIPQ_I32)
            return fail(HIPQ_ERR_UNSUPPORTED, "quantized type must be u8, i8 or i32");
        return HIPQ_OK;
    }

    static DimInfo dim_info(const hipq_quant_desc_t& d)
    {
        DimInfo di;
        di.rank = d.rank;
        di.axes_mask = d.axes_mask;
        for (int i = 0; i < HIPQ_MAX_RANK; ++i)
            di.shape[i] = i < d.rank ? d.shape[i] : 1;
        return di;
    }

    static unsigned generic_blocks(int64_t count)
    {
        int64_t b = (count + 255) / 256;
        return static_cast<unsigned>(b > 65536 ? 65536 : (b < 1 ? 1 : b));
    }

    static bool vec4_ok(const hipq_quant_desc_t& d, const Canon& c, const void* f32_ptr, const void* q_ptr)
    {
        return d.real_t == HIPQ_F32 && (d.quant_t == HIPQ_U8 || d.quant_t == HIPQ_I8) && c.single_run &&
               c.count < (1ll << 31) && c.count % 4 == 0 && (c.a == 1 || c.inner % 4 == 0) &&
               (reinterpret_cast<uintptr_t>(f32_ptr) & 15) == 0 && (reinterpret_cast<uintptr_t>(q_ptr) & 3) == 0;
    }

    // every 256-group step of a workgroup lies inside one row of the scale table
    static bool row_uniform(const Canon& c) { return c.a == 1 || (c.inner / 4) % 256 == 0; }

    static RunView make_view(const Canon& c)
    {
        RunView v;
        v.a = static_cast<uint32_t>(c.a);
        v.div_inner4 = make_fastdiv(static_cast<uint32_t>(c.a == 1 ? 1 : c.inner / 4));
        v.div_a = make_fastdiv(v.a);
        return v;
    }
}

using namespace hipq;

extern "C" {

int hipq_quantize(const hipq_quant_desc_t* d, const void* in, const void* scale, const void* zp, void* out, void* stream)
{
    int rc = check_desc(d);
    if (rc)
        return rc;
    HIPQ_REQUIRE(d->round_mode >= 0 && d->round_mode <= HIPQ_ROUND_DOWN, "round mode %d unknown", d->round_mode);
    Canon c = canonicalise(*d);
    if (c.count == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && scale && zp && out, "null tensor pointer");
    hipStream_t s = as_stream(stream);
    if (vec4_ok(*d, c, in, out))
    {
        uint32_t groups = static_cast<uint32_t>(c.count / 4);
        unsigned blocks = (groups + 256 * kQuantUnroll - 1) / (256 * kQuantUnroll);
        RunView v = make_view(c);
        bool rne = d->round_mode == HIPQ_ROUND_NEAREST_TOWARD_EVEN;
        bool uniform = row_uniform(c);
#define LAUNCH_Q4(QT, RNE, UNI)                                                                    \
    quantize_vec4_kernel<QT, RNE, UNI><<<blocks, 256, 0, s>>>(static_cast<const f32x4*>(in),      \
                                                              static_cast<const float*>(scale),    \
                                                              static_cast<const QT*>(zp),          \
                                                              static_cast<uint32_t*>(out),         \
                                                              groups,                              \
                                                              v,                                   \
                                                              d->round_mode)
#define LAUNCH_Q4_T(QT)                                                                            \
    do                                                                                             \
    {                                                                                              \
        if (rne && uniform)                                                                        \
            LAUNCH_Q4(QT, true, true);                                                             \
        else if (rne)                                                                              \
            LAUNCH_Q4(QT, true, false);                                                            \
        else if (uniform)                                                                          \
            LAUNCH_Q4(QT, false, true);                                                            \
        else                                                                                       \
            LAUNCH_Q4(QT, false, false);                                                           \
    } while (0)
        if (d->quant_t == HIPQ_I8)
            LAUNCH_Q4_T(int8_t);
        else
            LAUNCH_Q4_T(uint8_t);
#undef LAUNCH_Q4_T
#undef LAUNCH_Q4
        return check_launch("quantize_vec4");
    }
    DimInfo di = dim_info(*d);
    unsigned blocks = generic_blocks(c.count);
#define LAUNCH_QG(RT, QT)                                                                          \
    quantize_generic_kernel<RT, QT><<<blocks, 256, 0, s>>>(static_cast<const RT*>(in),             \
                                                           static_cast<const RT*>(scale),          \
                                                           static_cast<const QT*>(zp),             \
                                                           static_cast<QT*>(out),                  \
                                                           c.count,                                \
                                                           di,                                     \
                                                           d->round_mode)
    if (d->real_t == HIPQ_F32)
    {
        if (d->quant_t == HIPQ_U8)
            LAUNCH_QG(float, uint8_t);
        else if (d->quant_t == HIPQ_I8)
            LAUNCH_QG(float, int8_t);
        else
            LAUNCH_QG(float, int32_t);
    }
    else
    {
        if (d->quant_t == HIPQ_U8)
            LAUNCH_QG(double, uint8_t);
        else if (d->quant_t == HIPQ_I8)
            LAUNCH_QG(double, int8_t);
        else
            LAUNCH_QG(double, int32_t);
    }
#undef LAUNCH_QG
    return check_launch("quantize_generic");
}

int hipq_dequantize(const hipq_quant_desc_t* d, const void* in, const void* scale, const void* zp, void* out, void* stream)
{
    int rc = check_desc(d);
    if (rc)
        return rc;
    Canon c = canonicalise(*d);
    if (c.count == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && scale && zp && out, "null tensor pointer");
    hipStream_t s = as_stream(stream);
    if (vec4_ok(*d, c, out, in))
    {
        uint32_t groups = static_cast<uint32_t>(c.count / 4);
        unsigned blocks = (groups + 256 * kDequantUnroll - 1) / (256 * kDequantUnroll);
        RunView v = make_view(c);
        bool uniform = row_uniform(c);
#define LAUNCH_D4(QT, UNI)                                                                         \
    dequantize_vec4_kernel<QT, UNI><<<blocks, 256, 0, s>>>(static_cast<const uint32_t*>(in),       \
                                                           static_cast<const float*>(scale),       \
                                                           static_cast<const QT*>(zp),             \
                                                           static_cast<f32x4*>(out),               \
                                                           groups,                                 \
                                                           v)
        if (d->quant_t == HIPQ_I8)
        {
            if (uniform)
                LAUNCH_D4(int8_t, true);
            else
                LAUNCH_D4(int8_t, false);
        }
        else
        {
            if (uniform)
                LAUNCH_D4(uint8_t, true);
            else
                LAUNCH_D4(uint8_t, false);
        }
#undef LAUNCH_D4
        return check_launch("dequantize_vec4");
    }
    DimInfo di = dim_info(*d);
    unsigned blocks = generic_blocks(c.count);
#define LAUNCH_DG(QT, RT)                                                                          \
    dequantize_generic_kernel<QT, RT><<<blocks, 256, 0, s>>>(static_cast<const QT*>(in),           \
                                                             static_cast<const RT*>(scale),        \
                                                             static_cast<const QT*>(zp),           \
                                                             static_cast<RT*>(out),                \
                                                             c.count,                              \
                                                             di)
    if (d->real_t == HIPQ_F32)
    {
        if (d->quant_t == HIPQ_U8)
            LAUNCH_DG(uint8_t, float);
        else if (d->quant_t == HIPQ_I8)
            LAUNCH_DG(int8_t, float);
        else
            LAUNCH_DG(int32_t, float);
    }
    else
    {
        if (d->quant_t == HIPQ_U8)
            LAUNCH_DG(uint8_t, double);
        else if (d->quant_t == HIPQ_I8)
            LAUNCH_DG(int8_t, double);
        else
            LAUNCH_DG(int32_t, double);
    }
#undef LAUNCH_DG
    return check_launch("dequantize_generic");
}
}
