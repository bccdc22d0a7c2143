// Internal declarations shared by the translation units of libhipq.so.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "../../include/hipq.h"

namespace hipq
{
    // ---- host-side error plumbing ------------------------------------------------------------
    int fail(int code, const char* fmt, ...);
    void set_last_kernel(const char* name);

#define HIPQ_HIP(call)                                                                             \
    do                                                                                             \
    {                                                                                              \
        hipError_t e_ = (call);                                                                    \
        if (e_ != hipSuccess)                                                                      \
            return ::hipq::fail(HIPQ_ERR_HIP, "%s failed: %s", #call, hipGetErrorString(e_));      \
    } while (0)

#define HIPQ_REQUIRE(cond, ...)                                                                    \
    do                                                                                             \
    {                                                                                              \
        if (!(cond))                                                                               \
            return ::hipq::fail(HIPQ_ERR_INVALID, __VA_ARGS__);                                    \
    } while (0)

    inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
    int check_launch(const char* kernel);
    int device_compute_units(); // compute units of the current device (cached per device; 256 when the query fails)

    // Grow-only device workspace, one per (device, stream): launches on different streams never
    // share a block, so callers that run on streams of their own may overlap.  Growing a block waits
    // for its stream and frees the old one.
    int workspace(size_t bytes, hipStream_t stream, void** ptr);
    // a second block per (device, stream) for reductions split over workgroups: zeroed tile counters
    // (kSplitCounterBytes of them) followed by `partial_bytes` for partial sums
    constexpr size_t kSplitCounterBytes = 64 * 1024;
    int split_workspace(size_t partial_bytes, hipStream_t stream, uint32_t** counters, void** partials);
    // frees the blocks of a stream that is about to be destroyed
    int release_stream_workspace(hipStream_t stream);

    // Between noalloc_begin() and noalloc_end() on a thread, workspace() and split_workspace() hand
    // out pieces of a fixed per-device array instead of allocating (sizes beyond it: HIPQ_ERR_LIMIT).
    // noalloc_begin() fails when the array's address cannot be resolved on the current device.
    constexpr size_t kScratchWorkspaceBytes = HIPQ_NOALLOC_LAYOUT_BYTES; // layout copies (transposed / padded / unrolled input)
    constexpr size_t kScratchSplitBytes = HIPQ_NOALLOC_SPLIT_BYTES;      // tile counters + partial sums
    constexpr size_t kScratchBytes = kScratchWorkspaceBytes + kScratchSplitBytes;
    int noalloc_begin();
    void noalloc_end();

    inline size_t dtype_size(int t)
    {
        switch (t)
        {
        case HIPQ_U8:
        case HIPQ_I8: return 1;
        case HIPQ_I32:
        case HIPQ_F32: return 4;
        case HIPQ_F64: return 8;
        default: return 0;
        }
    }

    inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

    // ---- convolution geometry normalised to three spatial dims ------------------------------------
    struct ConvGeom
    {
        int64_t N, C, K;
        int64_t in[3], f[3], out[3], st[3], dl[3], dd[3], pb[3];
        int data_t, filter_t, out_t, data_layout, out_layout;
        __host__ __device__ int64_t out_count() const { return N * K * out[0] * out[1] * out[2]; }
        __host__ __device__ int64_t in_count() const { return N * C * in[0] * in[1] * in[2]; }
        __host__ __device__ int64_t taps() const { return f[0] * f[1] * f[2]; }
    };
    int make_geom(const hipq_conv_desc_t* d, ConvGeom* g);

    // ---- requantization epilogue, passed to kernels by value ----------------------------------
    enum
    {
        EPI_INTERP = 0, // INTERPRETER: half away from zero, narrowing wraps
        EPI_FUSED = 1   // oneDNN: bias, scale, sum, relu, half to even, saturate
    };

    struct Epilogue
    {
        int mode;
        int out_t;
        // EPI_INTERP: device scalars; scale = (*s_data * *s_filter) / *s_out
        const float* s_data;
        const float* s_filter;
        const float* s_out;
        const void* out_zp;
        // EPI_FUSED
        const int32_t* bias; // may be null
        const float* scale;  // [scale_count]
        const float* sum_scale;
        const void* sum_in; // may be null; indexed like out
        int sum_t;
        int relu;
        int per_channel; // scale_count > 1
        // EPI_FUSED with out_t F32, optional: the result goes through Gelu and Quantize (one scale and
        // zero point, device scalars) and only the quantized tensor is written
        const float* post_scale; // null: none
        const void* post_zp;
        int post_t;    // HIPQ_I8 / HIPQ_U8
        int post_mode; // round mode of the Quantize
    };

    // zero points of the accumulation, device scalars typed like their tensors (null = 0)
    struct ZeroPoints
    {
        const void* data_zp;
        const void* filter_zp;
        int data_t;
        int filter_t;
    };

#if defined(__HIPCC__)
    __device__ __forceinline__ int32_t load_q(const void* p, int t, size_t i)
    {
        switch (t)
        {
        case HIPQ_U8: return static_cast<const uint8_t*>(p)[i];
        case HIPQ_I8: return static_cast<const int8_t*>(p)[i];
        default: return static_cast<const int32_t*>(p)[i];
        }
    }

    __device__ __forceinline__ int32_t load_zp(const void* p, int t)
    {
        return p ? load_q(p, t, 0) : 0;
    }

    // float -> int32 the way x86 cvttss2si does it: NaN and out-of-range give INT32_MIN
    __device__ __forceinline__ int32_t cvtt_x86(float v)
    {
        if (!(v < 2147483648.0f) || v < -2147483648.0f)
            return INT32_MIN;
        return static_cast<int32_t>(v);
    }

    // Resolved per-thread view of an Epilogue (scalars loaded once).
    struct EpiRegs
    {
        float scale;     // interp scale, or fused scalar scale
        float sum_scale; // fused
        int32_t ozp;     // interp
    };

    __device__ __forceinline__ EpiRegs epi_load(const Epilogue& e)
    {
        EpiRegs r;
        r.sum_scale = 0.0f;
        r.ozp = 0;
        if (e.mode == EPI_INTERP)
        {
            // src/ngraph/runtime/reference/convolution.hpp:254 : two f32 roundings, this order
            r.scale = __fdiv_rn(__fmul_rn(*e.s_data, *e.s_filter), *e.s_out);
            r.ozp = load_zp(e.out_zp, e.out_t);
        }
        else
        {
            r.scale = e.scale[0];
            if (e.sum_in)
                r.sum_scale = *e.sum_scale;
        }
        return r;
    }

    // acc -> output value as int32 bits (for F32 outputs: the float's bit pattern).
    // k = output channel (bias / per-channel scale index), idx = flat output index (sum_in index).
    __device__ __forceinline__ int32_t epi_apply(const Epilogue& e, const EpiRegs& r, int32_t acc, int64_t k, int64_t idx)
    {
        if (e.mode == EPI_INTERP)
        {
            float v = roundf(__fmul_rn(static_cast<float>(acc), r.scale));
            int32_t t = cvtt_x86(v);
            if (e.out_t == HIPQ_U8)
                t = t & 0xFF;
            else if (e.out_t == HIPQ_I8)
                t = static_cast<int8_t>(t);
            return static_cast<int32_t>(static_cast<uint32_t>(t) + static_cast<uint32_t>(r.ozp));
        }
        float v = static_cast<float>(acc);
        if (e.bias)
            v = __fadd_rn(v, static_cast<float>(e.bias[k]));
        v = __fmul_rn(v, e.per_channel ? e.scale[k] : r.scale);
        if (e.sum_in)
            v = fmaf(r.sum_scale, static_cast<float>(load_q(e.sum_in, e.sum_t, idx)), v);
        if (e.relu)
            v = (v > 0.0f) ? v : __fmul_rn(v, -0.0f);
        if (e.out_t == HIPQ_F32)
            return __float_as_int(v);
        float lo = (e.out_t == HIPQ_U8) ? 0.0f : (e.out_t == HIPQ_I8 ? -128.0f : -2147483648.0f);
        float hi = (e.out_t == HIPQ_U8) ? 255.0f : (e.out_t == HIPQ_I8 ? 127.0f : 2147483520.0f);
        v = (v < lo) ? lo : v;
        v = (hi < v) ? hi : v;
        return static_cast<int32_t>(rintf(v));
    }

    __device__ __forceinline__ void store_out(void* out, int out_t, int64_t idx, int32_t v)
    {
        if (out_t == HIPQ_U8 || out_t == HIPQ_I8)
            static_cast<uint8_t*>(out)[idx] = static_cast<uint8_t>(v);
        else
            static_cast<int32_t*>(out)[idx] = v;
    }
#endif

    // ---- launchers implemented in the kernel translation units (host side) ------------------
    int launch_conv_direct(const ConvGeom& g,
                           const void* data,
                           const void* filter,
                           const ZeroPoints& zp,
                           const Epilogue& epi,
                           void* out,
                           hipStream_t s);
    int launch_dot_direct(const hipq_dot_desc_t& d,
                          const void* a,
                          const void* b,
                          const ZeroPoints& zp,
                          const Epilogue& epi,
                          void* out,
                          hipStream_t s);

    // MFMA implicit-GEMM convolution on channels-last data (both data and out NXC).
    bool conv_mfma_eligible(const ConvGeom& g);
    bool conv_band_eligible(const ConvGeom& g, bool out_ncx);
    int launch_conv_band(const ConvGeom& g,
                         const void* data_nxc,
                         const void* packed,
                         const ZeroPoints& zp,
                         const Epilogue& epi,
                         void* out,
                         bool out_ncx,
                         hipStream_t s);
    // 3x3 over 64 channels, filter in registers; data in the layout g.data_layout names
    bool conv_regw_eligible(const ConvGeom& g, bool out_ncx);
    int launch_conv_regw(const ConvGeom& g, const void* data, const void* packed, const ZeroPoints& zp, const Epilogue& epi, void* out, bool out_ncx, hipStream_t s);
    int launch_conv_mfma(const ConvGeom& g,
                         const void* data_nxc,
                         const void* packed,
                         const ZeroPoints& zp,
                         const Epilogue& epi,
                         void* out,
                         bool out_ncx, // false: out is channels-last; true: out is NCHW (written directly)
                         hipStream_t s);
    bool dot_mfma_eligible(const hipq_dot_desc_t& d);
    int launch_dot_mfma(const hipq_dot_desc_t& d,
                        const void* a,
                        const void* w_nk,      // [N,K] weights
                        const int32_t* wsum,   // [N]
                        const ZeroPoints& zp,
                        const Epilogue& epi,
                        void* out,
                        hipStream_t s,
                        const void* w_frag = nullptr); // fragment-ordered copy of the weights (prepacked blobs), or null

    int launch_rows_mfma(const void* a, bool a_unsigned, const int8_t* w_nk, const int32_t* wsum, int64_t M, int32_t N, int32_t K,
                         const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s, const char* name);

    int launch_rows_gelu_q8(const void* a, bool a_unsigned, const int8_t* w_nk, const int32_t* wsum, int64_t M, int32_t N, int32_t K, const ZeroPoints& zp, const Epilogue& epi,
                            void* out, hipStream_t s);

    int launch_transpose(const void* in, void* out, int64_t N, int64_t R, int64_t Cc, int elem_bytes, hipStream_t s);
    int launch_pad_channels(const void* in, void* out, int64_t N, int64_t X, int64_t Cc, bool in_ncx, const void* zp, int zp_t, hipStream_t s);
    bool conv_pad_eligible(const ConvGeom& g, ConvGeom* padded);
    int launch_im2col_nxc(const ConvGeom& g, const void* x_nxc, void* a, const void* zp, int zp_t, hipStream_t s);
    // first layers (at most four channels): staged copy with materialised padding + row-packed filter
    struct RowPack
    {
        int64_t Hp, Wp; // staged image extent
        int64_t kp;     // packed reduction bytes per output channel: filter rows x 32, rounded up to 64
    };
    bool conv_rowpack_eligible(const ConvGeom& g, RowPack* rp);
    int launch_stage_rows(const ConvGeom& g, const RowPack& rp, const void* in, void* staged, const void* zp, int zp_t, hipStream_t s);
    int launch_conv_rowpack(const ConvGeom& g, const RowPack& rp, const void* staged, const void* packed, const ZeroPoints& zp, const Epilogue& epi, void* out, hipStream_t s);
    // first layers with 64 output channels and a stride of two along the rows of pixels, fused
    // policy, u8 output: the band kernel that reads [N][C][H][W] bytes itself, and optionally reduces
    // a MaxPool over its own output before anything is written (hipq_conv_stem.hip)
    struct PoolFuse
    {
        int64_t wh, ww, sh, sw; // window, strides
        int64_t pt, pl;         // padding above / left
        int64_t out_h, out_w;   // extent of the pooled result
    };
    bool conv_stem_eligible(const ConvGeom& g, const Epilogue& epi, const ZeroPoints& zp, const PoolFuse* pool);
    int launch_conv_stem(const ConvGeom& g, const void* data, const void* packed, const ZeroPoints& zp, const Epilogue& epi, const PoolFuse* pool, void* out, hipStream_t s);
    // 1 x 1 layers from 64 to a multiple of 256 channels over many pixels, fused policy, channels-last:
    // weights in registers, tile loads one tile ahead (hipq_conv_pw.hip)
    bool conv_pw64_eligible(const ConvGeom& g, const Epilogue& epi, const ZeroPoints& zp);
    int launch_conv_pw64(const ConvGeom& g, const void* data, const void* packed, const Epilogue& epi, void* out, hipStream_t s);
    int launch_row_sums_i8(const void* w, int64_t rows, int64_t cols, int32_t* sums, hipStream_t s);
    // [N][K] weights in the fragment order of v_mfma_i32_16x16x64_i8 (K a multiple of 64): ceil(N / 16) * K / 64 blocks of 1 KB
    int launch_pack_dot_fragments(const void* w_nk, int64_t N, int64_t K, void* frag, hipStream_t s);
    // whether a packed blob of this product carries the fragment-ordered copy, and its size
    bool dot_fragments_eligible(const hipq_dot_desc_t& d);
    size_t dot_fragment_bytes(const hipq_dot_desc_t& d);
}
