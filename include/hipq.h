/*
 * hipq.h -- C ABI of libhipq.so: the int8 quantized-inference kernels for AMD gfx950 (MI355X).
 *
 * This is the seam between the C++ host side (the nGraph "HIP" backend plugin, which never includes
 * a HIP header) and the hand-written HIP kernels.  Every entry point takes plain pointers and
 * sizes; pointers named data/filter/out/scale/... are DEVICE pointers unless a comment says host.
 * All functions return HIPQ_OK (0) or an error code; hipq_last_error() gives the message of the
 * last failure on the calling thread.  A launch is asynchronous on `stream` (a hipStream_t passed
 * as void*, NULL = the default stream of the current device).
 *
 * Each compute entry point replaces one kernel of the nGraph reference and keeps its arithmetic.
 * Paths cited below are relative to the nGraph source tree.
 */
#ifndef HIPQ_H
#define HIPQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(_WIN32)
#define HIPQ_API
#else
#define HIPQ_API __attribute__((visibility("default")))
#endif

/* ---------------------------------------------------------------- status */
enum
{
    HIPQ_OK = 0,
    HIPQ_ERR_INVALID = 1,     /* malformed argument (null pointer, bad rank, shape mismatch) */
    HIPQ_ERR_UNSUPPORTED = 2, /* element-type combination the reference has no kernel for either */
    HIPQ_ERR_HIP = 3,         /* a HIP runtime call failed */
    HIPQ_ERR_LIMIT = 4        /* size beyond a documented maximum */
};

/* element types; the quantized ones are u8, i8, i32 (src/ngraph/type/element_type.cpp:83-88) */
typedef enum
{
    HIPQ_U8 = 0,
    HIPQ_I8 = 1,
    HIPQ_I32 = 2,
    HIPQ_F32 = 3,
    HIPQ_F64 = 4
} hipq_dtype_t;

/* same order as op::v0::Quantize::RoundMode (src/ngraph/op/quantize.hpp:38-81) */
typedef enum
{
    HIPQ_ROUND_NEAREST_TOWARD_INFINITY = 0,
    HIPQ_ROUND_NEAREST_TOWARD_ZERO = 1,
    HIPQ_ROUND_NEAREST_UPWARD = 2,
    HIPQ_ROUND_NEAREST_DOWNWARD = 3,
    HIPQ_ROUND_NEAREST_TOWARD_EVEN = 4,
    HIPQ_ROUND_TOWARD_INFINITY = 5,
    HIPQ_ROUND_TOWARD_ZERO = 6,
    HIPQ_ROUND_UP = 7,
    HIPQ_ROUND_DOWN = 8
} hipq_round_mode_t;

/* tensor layouts for convolution data / output.  NCX is the reference's (batch, channel,
 * spatial...) order; NXC is channels-last, the order the MFMA kernels consume natively. */
typedef enum
{
    HIPQ_LAYOUT_NCX = 0,
    HIPQ_LAYOUT_NXC = 1
} hipq_layout_t;

#define HIPQ_MAX_RANK 8
#define HIPQ_MAX_SPATIAL 3

/* ---------------------------------------------------------------- runtime plumbing */

typedef struct hipq_device_info
{
    char name[64];
    char arch[32];           /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
    int32_t compute_units;   /* CUs */
    int32_t clock_mhz;       /* peak engine clock */
    int32_t lds_bytes_per_cu;
    int32_t reserved;
    uint64_t hbm_bytes;      /* total device memory */
} hipq_device_info_t;

HIPQ_API const char* hipq_last_error(void);
HIPQ_API int hipq_version(void);
HIPQ_API int hipq_device_count(int* count);
HIPQ_API int hipq_set_device(int ordinal);
HIPQ_API int hipq_get_device_info(hipq_device_info_t* info);
HIPQ_API int hipq_malloc(void** dptr, size_t bytes);
HIPQ_API int hipq_free(void* dptr);
HIPQ_API int hipq_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes, void* stream);
HIPQ_API int hipq_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes, void* stream);
HIPQ_API int hipq_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes, void* stream);
/* byte fill done by a kernel (not a memset node), safe to record into a HIP graph */
HIPQ_API int hipq_fill_bytes(void* dst_dev, int value, size_t bytes, void* stream);
HIPQ_API int hipq_stream_create(void** stream);
HIPQ_API int hipq_stream_destroy(void* stream);
/* The library keeps grow-only scratch blocks per (device, stream) for every stream it has seen in a
 * call, its own or the caller's.  hipq_stream_destroy releases the blocks of a stream the library
 * created; a caller that passes streams of its own calls hipq_stream_release_scratch(stream) before
 * hipStreamDestroy (waits for the stream, frees its blocks, moves hipq_workspace_epoch): otherwise
 * the blocks stay until the process ends and a later stream with the same handle inherits them. */
HIPQ_API int hipq_stream_release_scratch(void* stream);
HIPQ_API int hipq_stream_sync(void* stream);
/* Stream capture into a HIP graph, for callers that replay one fixed launch sequence (what
 * runtime::Executable::call does, src/ngraph/runtime/executable.hpp:44-52): begin, issue the launches
 * on `stream` as usual (nothing runs), end -> an executable graph; hipq_graph_launch replays it on a
 * stream.  The launches between begin and end must not grow the per-device workspace: run the
 * sequence once uncaptured first.  hipq_workspace_epoch changes whenever the workspace of the
 * current device is reallocated; a graph captured under an older epoch may point into freed memory
 * and must be captured again. */
HIPQ_API int hipq_capture_begin(void* stream);
HIPQ_API int hipq_capture_end(void* stream, void** graph_exec);
HIPQ_API int hipq_graph_launch(void* graph_exec, void* stream);
HIPQ_API int hipq_graph_destroy(void* graph_exec);
HIPQ_API uint64_t hipq_workspace_epoch(void);
HIPQ_API int hipq_event_create(void** event);
HIPQ_API int hipq_event_destroy(void* event);
HIPQ_API int hipq_event_record(void* event, void* stream);
HIPQ_API int hipq_event_sync(void* event);
HIPQ_API int hipq_event_elapsed_ms(void* start, void* stop, float* ms);

/* ---------------------------------------------------------------- Quantize / Dequantize */

/*
 * Shape of the real/quantized tensor plus the axes the scale / zero-point tensors are laid along:
 * bit a of axes_mask set <=> axis a is in the op's AxisSet.  scale and zero_point are dense
 * row-major tensors whose shape is `shape` restricted to those axes (scalar when axes_mask == 0).
 */
typedef struct hipq_quant_desc
{
    int32_t real_t;     /* HIPQ_F32 or HIPQ_F64: input of quantize / output of dequantize */
    int32_t quant_t;    /* HIPQ_U8, HIPQ_I8 or HIPQ_I32 */
    int32_t rank;       /* 0..HIPQ_MAX_RANK */
    int32_t round_mode; /* hipq_round_mode_t; quantize only */
    uint32_t axes_mask;
    uint32_t reserved;
    int64_t shape[HIPQ_MAX_RANK];
} hipq_quant_desc_t;

/*
 * out = (QUANT) clamp(round_mode(in / scale[j]) + zero_point[j])        j = coordinate on `axes`
 * Replaces runtime::reference::quantize<REAL,QUANT>
 * (src/ngraph/runtime/reference/quantize.hpp:29-117, dispatched at
 * src/ngraph/runtime/interpreter/int_executable.hpp:1405-1451).
 * scale has type real_t, zero_point has type quant_t.  Bit-exact with the reference for finite
 * inputs (true IEEE division, the reference's floor/ceil rounding formulas, clamp in REAL).
 */
HIPQ_API int hipq_quantize(const hipq_quant_desc_t* desc,
                           const void* in,
                           const void* scale,
                           const void* zero_point,
                           void* out,
                           void* stream);

/*
 * out = (REAL)(in - zero_point[j]) * scale[j]
 * Replaces runtime::reference::dequantize<QUANT,REAL>
 * (src/ngraph/runtime/reference/dequantize.hpp:31-53, dispatched at int_executable.hpp:830-863).
 */
HIPQ_API int hipq_dequantize(const hipq_quant_desc_t* desc,
                             const void* in,
                             const void* scale,
                             const void* zero_point,
                             void* out,
                             void* stream);

/* ---------------------------------------------------------------- QuantizedConvolution */

typedef struct hipq_conv_desc
{
    int32_t n_spatial;   /* 1..HIPQ_MAX_SPATIAL */
    int32_t data_t;      /* HIPQ_U8 (the reference's only data type) or HIPQ_I8 */
    int32_t filter_t;    /* HIPQ_I8 or HIPQ_U8 */
    int32_t out_t;       /* HIPQ_I8, HIPQ_U8 or HIPQ_I32 */
    int32_t data_layout; /* hipq_layout_t of `data` (and of `sum_in`) */
    int32_t out_layout;  /* hipq_layout_t of `out` */
    int64_t N, C, K;     /* batch, input channels, output channels; filter is always K,C,spatial */
    int64_t in_sp[HIPQ_MAX_SPATIAL];
    int64_t f_sp[HIPQ_MAX_SPATIAL];
    int64_t out_sp[HIPQ_MAX_SPATIAL]; /* must equal hipq_conv_infer_output()'s result */
    int64_t stride[HIPQ_MAX_SPATIAL];        /* window_movement_strides */
    int64_t dilation[HIPQ_MAX_SPATIAL];      /* window_dilation_strides */
    int64_t data_dilation[HIPQ_MAX_SPATIAL]; /* data_dilation_strides */
    int64_t pad_below[HIPQ_MAX_SPATIAL];     /* may be negative */
    int64_t pad_above[HIPQ_MAX_SPATIAL];
} hipq_conv_desc_t;

/* Fills desc->out_sp with the reference's inferred output extent:
 * ((in-1)*data_dilation+1 + pad_below + pad_above - ((f-1)*dilation+1)) / stride + 1
 * (infer_convolution_forward, src/ngraph/validation_util.cpp).  HIPQ_ERR_INVALID if not positive. */
HIPQ_API int hipq_conv_infer_output(hipq_conv_desc_t* desc);

/*
 * Prepacked filter for the MFMA path.  hipq_conv_packed_filter_bytes returns 0 when the shape /
 * type combination is not eligible for that path (the call then runs on the direct kernel and
 * `packed` may be NULL).  The packed blob holds the filter reordered to K,spatial,C plus a
 * per-output-channel table of sum(filter) used to run u8 data on the signed i8 MFMA.
 * Pass the blob to a convolution call only when the filter zero point is zero (the nGraph CPU
 * backend makes the same demand of its fast path, src/ngraph/runtime/cpu/pass/cpu_assignment.cpp:
 * 801-825); a non-zero one is still computed correctly, by a slow in-kernel path.
 */
HIPQ_API size_t hipq_conv_packed_filter_bytes(const hipq_conv_desc_t* desc);
HIPQ_API int hipq_conv_pack_filter(const hipq_conv_desc_t* desc,
                                   const void* filter,
                                   void* packed,
                                   void* stream);

/*
 * op::v0::QuantizedConvolution.  Replaces runtime::reference::convolution<IN,FILT,OUT,int32_t>
 * (src/ngraph/runtime/reference/convolution.hpp:55-265,267-313; dispatched at
 * int_executable.hpp:1453-1558) with the INTERPRETER's arithmetic:
 *   acc   = sum over in-bounds taps of (data - *data_zp) * (filter - *filter_zp)      int32
 *   scale = (*data_scale * *filter_scale) / *out_scale                                f32
 *   out   = (OUT) roundf((float)acc * scale) + *out_zp      half away from zero, narrowing wraps
 * The six scale / zero-point arguments are DEVICE pointers to scalars (they may be graph
 * Parameters), zero points typed like the tensor they belong to.
 */
HIPQ_API int hipq_quantized_convolution(const hipq_conv_desc_t* desc,
                                        const void* data,
                                        const void* filter,
                                        const void* packed_filter, /* may be NULL */
                                        const float* data_scale,
                                        const void* data_zp,
                                        const float* filter_scale,
                                        const void* filter_zp,
                                        const float* out_scale,
                                        const void* out_zp,
                                        void* out,
                                        void* stream);

/*
 * hipq_quantized_convolution for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the nGraph
 * reference.  Arguments, kernels and results are those of hipq_quantized_convolution; the difference
 * is where scratch comes from.  That entry point keeps grow-only blocks per stream (hipMalloc on
 * first use and on growth); this one calls no hipMalloc / hipFree at all and takes its scratch from
 * a fixed array that every GPU the library runs on holds from load time until the process ends:
 *   HIPQ_NOALLOC_LAYOUT_BYTES  for the channels-last / padded / unrolled copy of an NCX input
 *                              (an NCX u8 input of up to that many bytes; channels-last inputs
 *                              with 64-multiple channel counts need none, nor do 3x3 stride-1
 *                              layers over 64 channels with an NCX output, whose kernel reads
 *                              NCX itself)
 *   HIPQ_NOALLOC_SPLIT_BYTES   for tile counters (64 KiB) and partial sums of reductions split over
 *                              workgroups
 * A call that would need more returns HIPQ_ERR_LIMIT and launches nothing.  Every call on a GPU
 * shares that GPU's array: calls of this entry point that overlap on one GPU (two streams, two
 * threads) race; calls on one stream are ordered by the stream.  The tile counters are cleared by
 * a kernel on `stream` ahead of every launch that uses them.
 * Set-up: hipq_set_device resolves the array's address on that device.  A caller that selects its
 * device some other way makes one call of this entry point outside any graph capture first (the
 * first call on a device resolves the address itself, which is not a step to record into a graph).
 */
#define HIPQ_NOALLOC_LAYOUT_BYTES (32u << 20)
#define HIPQ_NOALLOC_SPLIT_BYTES (16u << 20)
HIPQ_API int hipq_quantized_convolution_noalloc(const hipq_conv_desc_t* desc,
                                                const void* data,
                                                const void* filter,
                                                const void* packed_filter, /* may be NULL */
                                                const float* data_scale,
                                                const void* data_zp,
                                                const float* filter_scale,
                                                const void* filter_zp,
                                                const float* out_scale,
                                                const void* out_zp,
                                                void* out,
                                                void* stream);

/* Post-ops of the fused ops.  The arithmetic is oneDNN's as driven by the nGraph CPU backend:
 *   v = scale[k or 0] * ((float)acc + (float)bias[k]);  v = fmaf(sum_scale, (float)sum_in, v);
 *   v = relu ? max(v, 0) : v;  out = saturate<OUT>(nearbyintf(v))        round-half-to-even
 */
typedef struct hipq_fused_desc
{
    int32_t has_bias;    /* bias: int32[K] */
    int32_t has_sum;     /* sum_in: tensor shaped and laid out like out */
    int32_t sum_t;       /* HIPQ_U8 or HIPQ_I8 (QuantizedConvolutionBiasSignedAdd reads i8) */
    int32_t with_relu;
    int64_t scale_count; /* 1, or K for per-output-channel requantization scales */
} hipq_fused_desc_t;

/*
 * op::v0::QuantizedConvolutionBias / ...Relu / ...BiasAdd / ...BiasSignedAdd
 * (src/ngraph/op/experimental/quantized_conv_bias.cpp:26-237, quantized_conv_relu.cpp:25-80;
 * executed by src/ngraph/runtime/cpu/builder/quantized_conv.cpp:332-766 with the attributes of
 * src/ngraph/runtime/cpu/dnnl_emitter.hpp:668-706).  data must be u8 or i8, filter i8, zero points
 * are all 0; out_t is desc->out_t.  sum_in may alias out.
 */
HIPQ_API int hipq_quantized_convolution_fused(const hipq_conv_desc_t* desc,
                                              const hipq_fused_desc_t* fused,
                                              const void* data,
                                              const void* filter,
                                              const void* packed_filter, /* may be NULL */
                                              const int32_t* bias,
                                              const void* sum_in,
                                              const float* scale,
                                              const float* sum_scale,
                                              void* out,
                                              void* stream);

/* ---------------------------------------------------------------- QuantizedDot */

typedef enum
{
    HIPQ_B_KN = 0, /* second operand is [K,N] row-major: op::v0::QuantizedDot */
    HIPQ_B_NK = 1  /* second operand is [N,K] row-major: op::v0::QuantizedDotBias weights */
} hipq_b_layout_t;

typedef struct hipq_dot_desc
{
    int32_t a_t;      /* HIPQ_U8 or HIPQ_I8 */
    int32_t b_t;      /* HIPQ_I8 or HIPQ_U8 */
    int32_t out_t;    /* HIPQ_I8, HIPQ_U8, HIPQ_I32, or HIPQ_F32 (QuantizedDotBias, no requantize) */
    int32_t b_layout; /* hipq_b_layout_t */
    int64_t M, K, N;
} hipq_dot_desc_t;

/*
 * Prepacked second operand for the MFMA path.  hipq_dot_packed_bytes returns 0 when the shape /
 * type combination is not eligible for that path.  The blob holds the operand as [N,K] (a
 * transposed copy for HIPQ_B_KN, nothing for HIPQ_B_NK, which is used in place) followed by a
 * table int32[N] of sum_k(b[k,n]) used to run u8 activations on the signed i8 MFMA.  Passing
 * NULL for `packed_b` makes the call build the same data in an internal workspace every time.
 * Like the packed filter, it is only valid while the second operand's zero point is zero.
 */
HIPQ_API size_t hipq_dot_packed_bytes(const hipq_dot_desc_t* desc);
HIPQ_API int hipq_dot_pack(const hipq_dot_desc_t* desc, const void* b, void* packed, void* stream);

/*
 * op::v0::QuantizedDot with one reduction axis.  Replaces runtime::reference::dot<IN0,IN1,OUT,int32_t>
 * (src/ngraph/runtime/reference/dot.hpp:34-167; dispatched at int_executable.hpp:1565-1653),
 * INTERPRETER arithmetic as for hipq_quantized_convolution.  a is [M,K], b is [K,N].
 */
HIPQ_API int hipq_quantized_dot(const hipq_dot_desc_t* desc,
                                const void* a,
                                const void* b,
                                const void* packed_b, /* may be NULL */
                                const float* a_scale,
                                const void* a_zp,
                                const float* b_scale,
                                const void* b_zp,
                                const float* out_scale,
                                const void* out_zp,
                                void* out,
                                void* stream);

/*
 * op::v0::QuantizedDotBias (src/ngraph/op/experimental/quantized_dot_bias.cpp:27-56; executed by
 * src/ngraph/runtime/cpu/builder/quantized_dot.cpp:36-125, attributes dnnl_emitter.hpp:737-761).
 * a is u8 or i8 [M,K], w is i8 [N,K], bias int32[N] (has_bias), scale f32[scale_count].
 * out_t F32: out = relu?(scale * (acc + bias));  I8/U8: saturate(nearbyint(that)).
 * has_sum must be 0.
 */
HIPQ_API int hipq_quantized_dot_bias(const hipq_dot_desc_t* desc,
                                     const hipq_fused_desc_t* fused,
                                     const void* a,
                                     const void* w,
                                     const void* packed_w, /* may be NULL */
                                     const int32_t* bias,
                                     const float* scale,
                                     void* out,
                                     void* stream);

/*
 * Quantize(Gelu(QuantizedDotBias(...) as f32)): the first projection of a transformer encoder's feed-forward
 * block with the activation and the Quantize that follow it, one launch where the kernels that load
 * straight into LDS take the product (more than 256 rows, more than 64 outputs in multiples of 16),
 * the product into the library's workspace and hipq_gelu_quantize_f32 otherwise.  desc->out_t must be
 * HIPQ_F32 (the form of the product); only quant->out ([M,N] bytes, 16-byte aligned, not overlapping a) is written, equal
 * bit for bit to hipq_quantized_dot_bias followed by hipq_gelu_quantize_f32.  hipq_quant_out_t is declared
 * with the fp32 glue below.  No counterpart as a single reference op
 * (src/ngraph/op/experimental/quantized_dot_bias.cpp:27-56, src/ngraph/op/gelu.cpp:46-60,
 * src/ngraph/runtime/reference/quantize.hpp:29-117).
 */
struct hipq_quant_out;
HIPQ_API int hipq_quantized_dot_bias_gelu_quantize(const hipq_dot_desc_t* desc,
                                                   const hipq_fused_desc_t* fused,
                                                   const void* a,
                                                   const void* w,
                                                   const void* packed_w, /* may be NULL where the fused kernels apply; needed otherwise */
                                                   const int32_t* bias,
                                                   const float* scale,
                                                   const struct hipq_quant_out* quant,
                                                   void* stream);

/* ---------------------------------------------------------------- layout helpers */

/* [N,C,X] -> [N,X,C] and back for elem_bytes in {1,4}; X = product of spatial extents. */
HIPQ_API int hipq_transpose_ncx_to_nxc(
    const void* in, void* out, int64_t N, int64_t C, int64_t X, int32_t elem_bytes, void* stream);
HIPQ_API int hipq_transpose_nxc_to_ncx(
    const void* in, void* out, int64_t N, int64_t C, int64_t X, int32_t elem_bytes, void* stream);

/* ---------------------------------------------------------------- glue ops
 * The small elementwise / shape ops that surround the quantized ops in a graph: the f32 scale
 * sub-graphs the builders emit (src/ngraph/builder/quantization_utils.cpp:33-174), and the integer
 * glue of quantized networks.  Arithmetic is the reference's (src/ngraph/runtime/reference/
 * {abs,relu,add,subtract,multiply,divide,maximum,minimum,convert,broadcast,reshape}.hpp): plain C++
 * operators on the element type, so 8-bit sums wrap and Convert is a static_cast. */
typedef enum
{
    HIPQ_OP_ADD = 0,
    HIPQ_OP_SUBTRACT = 1,
    HIPQ_OP_MULTIPLY = 2,
    HIPQ_OP_DIVIDE = 3,
    HIPQ_OP_MAXIMUM = 4,
    HIPQ_OP_MINIMUM = 5,
    HIPQ_OP_DIVIDE_FLOOR = 6
} hipq_binary_op_t;
/* HIPQ_OP_DIVIDE is op::v1::Divide with is_pythondiv() false (C++ truncation), HIPQ_OP_DIVIDE_FLOOR
 * with it true, the op's default (src/ngraph/op/divide.hpp:72,
 * src/ngraph/runtime/reference/divide.hpp:41-60: quotient less one when the remainder is not zero
 * and the signs differ); floating types divide the same way under both.  Deviation: the reference
 * throws std::domain_error on an integer zero divisor; a kernel cannot throw, the element is 0. */

typedef enum
{
    HIPQ_OP_ABS = 0,
    HIPQ_OP_RELU = 1,
    HIPQ_OP_COPY = 2
} hipq_unary_op_t;

/* out[i] = a[i or 0] (op) b[i or 0]; a_count and b_count are each `count` or 1 (broadcast scalar) */
HIPQ_API int hipq_binary(int32_t op,
                         int32_t dtype,
                         const void* a,
                         int64_t a_count,
                         const void* b,
                         int64_t b_count,
                         void* out,
                         int64_t count,
                         void* stream);
HIPQ_API int hipq_unary(int32_t op, int32_t dtype, const void* in, void* out, int64_t count, void* stream);
/* out[i] = static_cast<OUT>(in[i]) with the x86 narrowing of the reference build */
HIPQ_API int hipq_convert(int32_t in_t, int32_t out_t, const void* in, void* out, int64_t count, void* stream);
/* op::v0::Broadcast: `in` has out_shape minus the axes in axes_mask */
HIPQ_API int hipq_broadcast(int32_t elem_bytes,
                            const void* in,
                            void* out,
                            int32_t out_rank,
                            const int64_t* out_shape, /* host */
                            uint32_t axes_mask,
                            void* stream);
/* op::v0::Reshape's transposition: out = in with axes read in `order` (out dim i = in dim order[i]) */
HIPQ_API int hipq_permute(int32_t elem_bytes,
                          const void* in,
                          void* out,
                          int32_t rank,
                          const int64_t* in_shape, /* host */
                          const int32_t* order,    /* host */
                          void* stream);

/* op::v0::Slice (src/ngraph/runtime/reference/slice.hpp:30-66): out[c] = in[lower + c * strides] along
 * every axis, out extent ceil((upper - lower) / strides); 0 <= lower <= upper <= extent. */
HIPQ_API int hipq_slice(int32_t elem_bytes,
                        const void* in,
                        void* out,
                        int32_t rank,
                        const int64_t* in_shape, /* host */
                        const int64_t* lower,    /* host */
                        const int64_t* upper,    /* host */
                        const int64_t* strides,  /* host */
                        void* stream);

/* ---- pooling and concatenation: the integer glue between the quantized convolutions of a network ----
 * MaxPool / AvgPool replace runtime::reference::max_pool<T> (src/ngraph/runtime/reference/
 * max_pool.hpp:127-222) and avg_pool<T> (src/ngraph/runtime/reference/avg_pool.hpp:128-250):
 * padding never wins a maximum (a window wholly in the padding gives the type's lowest value); the
 * average sums in the element type -- an 8-bit sum wraps -- and for 8-bit types is
 * nearbyint(float(sum) / count), ties to even; padding enters sum and count only when
 * include_padding is set.  Types: u8, i8, f32, and i32 for MaxPool. */
typedef enum
{
    HIPQ_POOL_MAX = 0,
    HIPQ_POOL_AVG = 1
} hipq_pool_op_t;

typedef struct
{
    int32_t op;              /* hipq_pool_op_t */
    int32_t dtype;           /* hipq_dtype_t */
    int32_t layout;          /* hipq_layout_t of input and output */
    int32_t n_spatial;       /* 1..HIPQ_MAX_SPATIAL */
    int32_t include_padding; /* AvgPool's include_padding_in_avg_computation */
    int64_t N, C;
    int64_t in_sp[HIPQ_MAX_SPATIAL];
    int64_t window[HIPQ_MAX_SPATIAL];
    int64_t stride[HIPQ_MAX_SPATIAL];
    int64_t pad_below[HIPQ_MAX_SPATIAL];
    int64_t pad_above[HIPQ_MAX_SPATIAL];
    int64_t out_sp[HIPQ_MAX_SPATIAL]; /* filled by hipq_pool_infer_output */
} hipq_pool_desc_t;

/* out_sp[i] = (in + pad_below + pad_above - window) / stride + 1, the rule of
 * infer_batched_pooling_forward (src/ngraph/validation_util.cpp) */
HIPQ_API int hipq_pool_infer_output(hipq_pool_desc_t* desc);
HIPQ_API int hipq_pool(const hipq_pool_desc_t* desc, const void* in, void* out, void* stream);

/*
 * MaxPool(QuantizedConvolutionBias(...)) in one launch, for the pairs a first layer makes: the
 * convolution is the one hipq_quantized_convolution_fused would run with these descriptors (no
 * residual input; src/ngraph/runtime/cpu/builder/quantized_conv.cpp:332-766), the pool the one
 * hipq_pool would run over its result (src/ngraph/runtime/reference/max_pool.hpp:127-222); `out`
 * is the pooled tensor and the convolution's own result is never written.  The bytes equal the two
 * calls'.  Eligible pairs (hipq_conv_max_pool_fusable returns 1): [N][C][H][W] u8 / i8 data with at
 * most four channels and a width that is a multiple of four, 64 output channels, a filter of up to
 * 8 x 8 taps with a column stride of two, u8 channels-last output, a pool window of up to 3 x 3.
 * `packed_filter` is required (hipq_conv_pack_filter); `data` must be 4-byte aligned.
 * HIPQ_ERR_UNSUPPORTED for any other pair: the caller then makes the two calls.
 */
HIPQ_API int hipq_conv_max_pool_fusable(const hipq_conv_desc_t* desc, const hipq_fused_desc_t* fused, const hipq_pool_desc_t* pool);
HIPQ_API int hipq_quantized_convolution_fused_max_pool(const hipq_conv_desc_t* desc,
                                                       const hipq_fused_desc_t* fused,
                                                       const hipq_pool_desc_t* pool,
                                                       const void* data,
                                                       const void* packed_filter,
                                                       const int32_t* bias,
                                                       const float* scale,
                                                       void* out,
                                                       void* stream);

/* op::v0::Concat (src/ngraph/runtime/reference/concat.hpp): piece i is [outer][extent[i]][inner]
 * elements, the result [outer][sum extent][inner]; `inputs` and `extents` are host arrays of
 * device pointers / axis extents. */
HIPQ_API int hipq_concat(int32_t elem_bytes,
                         int32_t n_inputs,
                         const void* const* inputs,
                         const int64_t* extents,
                         int64_t outer,
                         int64_t inner,
                         void* out,
                         void* stream);

/* ---- fp32 glue of a transformer encoder (between the quantized projections) ----------------------
 * Floating point: results agree with the reference's to 1e-5 relative (the reference sums
 * sequentially with Kahan compensation, src/ngraph/runtime/reference/sum.hpp:56-88, and calls the
 * host's expf / erff; the kernels reduce in parallel and call the device's). */

/* op::v0::Softmax over a contiguous run of axes, the tensor seen as [outer][axis][inner]:
 * out = exp(x - max) / sum(exp(x - max)) along `axis`
 * (src/ngraph/runtime/reference/softmax.hpp:31-57). */
HIPQ_API int hipq_softmax_f32(const float* in, float* out, int64_t outer, int64_t axis, int64_t inner, void* stream);

/* Softmax(Multiply(in, Broadcast(factor))) in one pass: `factor` is a device f32 scalar, every
 * product is rounded to f32 as op::v1::Multiply rounds it (src/ngraph/runtime/reference/multiply.hpp),
 * so the result equals hipq_binary(multiply) followed by hipq_softmax_f32 bit for bit.  What an
 * attention layer's scores / sqrt(head size) -> Softmax chain lowers to. */
HIPQ_API int hipq_softmax_scaled_f32(const float* in, const float* factor, float* out, int64_t outer, int64_t axis, int64_t inner, void* stream);

/* A Quantize of a kernel's f32 result, written beside it (one scale and zero point for the whole
 * tensor; arithmetic of hipq_quantize, src/ngraph/runtime/reference/quantize.hpp:29-117, so the bytes
 * equal a hipq_quantize call on the f32 result).  What a backend passes when the only consumer of an
 * f32 tensor -- or one of two -- is a Quantize: the tensor is not read back from memory for it. */
typedef struct hipq_quant_out
{
    void* out;              /* [same element count], quant_t */
    const float* scale;     /* device scalar */
    const void* zero_point; /* device scalar of quant_t; null: 0 */
    int32_t quant_t;        /* HIPQ_I8 or HIPQ_U8 */
    int32_t round_mode;     /* hipq_round_mode_t */
} hipq_quant_out_t;

/* op::v0::Erf (src/ngraph/runtime/reference/erf.hpp:29-35). */
HIPQ_API int hipq_erf_f32(const float* in, float* out, int64_t count, void* stream);

/* op::v0::Gelu as FusedOpDecomposition lowers it (src/ngraph/op/gelu.cpp:46-60):
 * (0.5 * x) * (1 + erf(x / sqrt(2))), every step in f32. */
HIPQ_API int hipq_gelu_f32(const float* in, float* out, int64_t count, void* stream);

/* Gelu with a Quantize of its result: q->out = Quantize(Gelu(in)); `out` (the f32 result) may be null
 * when the Quantize is its only consumer.  Equals hipq_gelu_f32 + hipq_quantize bit for bit. */
HIPQ_API int hipq_gelu_quantize_f32(const float* in, float* out, const hipq_quant_out_t* q, int64_t count, void* stream);

/* op::v0::LayerNorm forward as it decomposes (src/ngraph/op/layer_norm.cpp:68-150,
 * src/ngraph/builder/reduce_ops.cpp:68-124): the tensor is [rows][cols] with cols the product of the
 * normalised trailing axes; mean = sum(x) / cols, var = sum((x - mean)^2) / cols,
 * out = (x - mean) / sqrt(var + epsilon) * scale + bias.  scale and bias ([cols]) may both be null
 * (use_affine = false); mean and var ([rows]) may be null (keep_stats = false). */
HIPQ_API int hipq_layer_norm_f32(const float* in,
                                 const float* scale,
                                 const float* bias,
                                 float* out,
                                 float* mean,
                                 float* var,
                                 int64_t rows,
                                 int64_t cols,
                                 double epsilon,
                                 void* stream);

/* LayerNorm(Add(a, b)) in one pass, optionally with a Quantize of the result beside it:
 * out = LayerNorm(a + b) (b may be null: LayerNorm(a)), the sum rounded to f32 as op::v1::Add rounds
 * it; q (may be null) as above.  Equals hipq_binary(add) + hipq_layer_norm_f32 (+ hipq_quantize) bit
 * for bit: the residual-and-normalise step of a transformer layer whose result feeds the next
 * quantized projection. */
HIPQ_API int hipq_add_layer_norm_f32(const float* a,
                                     const float* b,
                                     const float* scale,
                                     const float* bias,
                                     float* out,
                                     const hipq_quant_out_t* q,
                                     int64_t rows,
                                     int64_t cols,
                                     double epsilon,
                                     void* stream);

/* op::v0::BatchMatMul (src/ngraph/runtime/reference/batch_mat_mul.hpp:31-57: runtime::reference::dot,
 * dot.hpp:34-167 with one reduction axis, on every pair of the batch), op::v0::Dot of two f32
 * matrices (batch = 1), and op::v0::BatchMatMulTranspose (src/ngraph/op/batch_mat_mul_transpose.hpp),
 * which reads either operand transposed: out[b] = op(a[b]) * op(b[b]), a[b] stored [M][K] (or [K][M]
 * with transpose_a), b[b] stored [K][N] (or [N][K] with transpose_b), out[b] [M][N].  The reference
 * accumulates in double, k ascending, and rounds once to f32 (dot.hpp:37: ACCUMULATION =
 * widen<float>::type, convolution.hpp:34-44); so does the kernel: the results are bit-exact. */
HIPQ_API int hipq_batch_matmul_f32(const float* a,
                                   const float* b,
                                   float* out,
                                   int64_t batch,
                                   int64_t M,
                                   int64_t K,
                                   int64_t N,
                                   int32_t transpose_a,
                                   int32_t transpose_b,
                                   void* stream);

/* The same product on views of larger tensors and into one, with an optional Quantize of the result:
 * batch element e = outer * batch_inner + inner reads a + outer * a_outer + inner * a_inner with
 * rows lda elements apart (likewise b and out; strides in elements, rows at least as far apart as
 * they are long).  What BatchMatMul(Reshape / transpose of a slice) lowers to without moving data:
 * the Q, K and V heads of a fused [tokens, 3 * hidden] projection, and a context written straight
 * into the [tokens, hidden] layout of the merged heads.  q (may be null): Quantize of the f32 result
 * at the same element offsets of q->out; `out` may then be null.  Bit-exact like the plain entry point;
 * no counterpart as a single reference op. */
typedef struct hipq_matmul_view
{
    int64_t batch_inner;
    int64_t a_outer, a_inner, lda;
    int64_t b_outer, b_inner, ldb;
    int64_t o_outer, o_inner, ldo;
} hipq_matmul_view_t;
HIPQ_API int hipq_batch_matmul_view_f32(const float* a,
                                        const float* b,
                                        float* out,
                                        const hipq_matmul_view_t* view,
                                        const hipq_quant_out_t* q,
                                        int64_t batch,
                                        int64_t M,
                                        int64_t K,
                                        int64_t N,
                                        int32_t transpose_a,
                                        int32_t transpose_b,
                                        void* stream);

/* Attention of a batch of heads in one launch:
 *   out = BatchMatMul(Softmax(Multiply(BatchMatMulTranspose(Q, K), *factor)), V)
 * -- the sub-graph between the QKV projection and the output projection of a transformer encoder
 * (src/ngraph/runtime/reference/batch_mat_mul.hpp:31-57, softmax.hpp:31-57, multiply.hpp), with
 * an optional Quantize of the result.  Equal, bit for bit, to hipq_batch_matmul_view_f32 (transpose_b),
 * hipq_softmax_scaled_f32 and hipq_batch_matmul_view_f32 in sequence; the [queries, keys] scores stay
 * on the compute unit.  Q is [queries, depth], K and V are [keys, depth] per batch element, addressed
 * like the views above (strides in elements); factor may be null (no Multiply); out may be null when
 * quant is given.  Returns HIPQ_ERR_UNSUPPORTED (nothing launched) unless keys == 128, depth == 64 and
 * queries is a multiple of 32: callers then run the three ops.  No counterpart as a single reference op. */
typedef struct hipq_attention_view
{
    int64_t batch_inner;
    int64_t q_outer, q_inner, ldq;
    int64_t k_outer, k_inner, ldk;
    int64_t v_outer, v_inner, ldv;
    int64_t o_outer, o_inner, ldo;
} hipq_attention_view_t;
HIPQ_API int hipq_attention_f32(const float* q,
                                const float* k,
                                const float* v,
                                const float* factor,
                                float* out,
                                const hipq_attention_view_t* view,
                                const hipq_quant_out_t* quant,
                                int64_t batch,
                                int64_t queries,
                                int64_t keys,
                                int64_t depth,
                                void* stream);

/* Which kernel the last hipq_quantized_* call on this thread used: "mfma", "direct", ... (host
 * string, never NULL).  For tests and profiles. */
HIPQ_API const char* hipq_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif /* HIPQ_H */
