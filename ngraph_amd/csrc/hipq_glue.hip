// Elementwise and shape glue around the quantized ops (tiny f32 scale tensors, integer glue).
#include "hipq_common.h"

namespace hipq
{
    // reference::divide with pythondiv (src/ngraph/runtime/reference/divide.hpp:41-60): the truncated
    // quotient, less one when the remainder is not zero and the signs differ.  Floating types have
    // no such mode: the reference divides them the same way whatever the flag says.
    template <typename T>
    __device__ __forceinline__ T floor_divide(T a, T b)
    {
        if constexpr (std::is_integral<T>::value)
        {
            const int32_t x = a, y = b; // 8-bit operands promote; int32 has a specialisation
            const int32_t quot = x / y, rem = x % y;
            return static_cast<T>((rem != 0 && ((x < 0) != (y < 0))) ? quot - 1 : quot);
        }
        else
            return static_cast<T>(a / b);
    }

    template <typename T>
    __device__ __forceinline__ T binary_apply(int op, T a, T b)
    {
        switch (op)
        {
        case HIPQ_OP_ADD: return static_cast<T>(a + b);
        case HIPQ_OP_SUBTRACT: return static_cast<T>(a - b);
        case HIPQ_OP_MULTIPLY: return static_cast<T>(a * b);
        case HIPQ_OP_DIVIDE: return static_cast<T>(a / b);
        case HIPQ_OP_DIVIDE_FLOOR: return floor_divide(a, b);
        case HIPQ_OP_MAXIMUM: return a > b ? a : b;
        default: return a < b ? a : b;
        }
    }
    template <>
    __device__ __forceinline__ float binary_apply<float>(int op, float a, float b)
    {
        switch (op)
        {
        case HIPQ_OP_ADD: return __fadd_rn(a, b);
        case HIPQ_OP_SUBTRACT: return __fsub_rn(a, b);
        case HIPQ_OP_MULTIPLY: return __fmul_rn(a, b);
        case HIPQ_OP_DIVIDE:
        case HIPQ_OP_DIVIDE_FLOOR: return __fdiv_rn(a, b);
        case HIPQ_OP_MAXIMUM: return a > b ? a : b;
        default: return a < b ? a : b;
        }
    }
    // Integer division by zero: the reference throws std::domain_error from the host loop; a kernel
    // cannot, so a zero divisor gives 0 (documented deviation).  INT32_MIN / -1 overflows in C++; the
    // x86 build of the reference traps on it, here it gives INT32_MIN.
    template <>
    __device__ __forceinline__ int32_t binary_apply<int32_t>(int op, int32_t a, int32_t b)
    {
        switch (op)
        {
        case HIPQ_OP_ADD: return static_cast<int32_t>(static_cast<uint32_t>(a) + static_cast<uint32_t>(b));
        case HIPQ_OP_SUBTRACT: return static_cast<int32_t>(static_cast<uint32_t>(a) - static_cast<uint32_t>(b));
        case HIPQ_OP_MULTIPLY: return static_cast<int32_t>(static_cast<uint32_t>(a) * static_cast<uint32_t>(b));
        case HIPQ_OP_DIVIDE: return b == 0 ? 0 : (a == INT32_MIN && b == -1 ? INT32_MIN : a / b);
        case HIPQ_OP_DIVIDE_FLOOR:
        {
            if (b == 0)
                return 0;
            if (a == INT32_MIN && b == -1)
                return INT32_MIN;
            const int32_t quot = a / b, rem = a % b;
            return (rem != 0 && ((a < 0) != (b < 0))) ? quot - 1 : quot;
        }
        case HIPQ_OP_MAXIMUM: return a > b ? a : b;
        default: return a < b ? a : b;
        }
    }

    template <typename T>
    __global__ __launch_bounds__(256) void binary_kernel(int op, const T* a, int64_t an, const T* b, int64_t bn, T* out, int64_t n)
    {
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < n; i += step)
        {
            T x = a[an == 1 ? 0 : i], y = b[bn == 1 ? 0 : i];
            if (sizeof(T) == 1 && (op == HIPQ_OP_DIVIDE || op == HIPQ_OP_DIVIDE_FLOOR) && y == 0)
                out[i] = 0;
            else
                out[i] = binary_apply<T>(op, x, y);
        }
    }

    template <typename T>
    __global__ __launch_bounds__(256) void unary_kernel(int op, const T* in, T* out, int64_t n)
    {
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < n; i += step)
        {
            T x = in[i];
            if (op == HIPQ_OP_ABS)
                out[i] = x < T(0) ? static_cast<T>(-x) : x; // reference::abs: (x < 0 ? -x : x)
            else if (op == HIPQ_OP_RELU)
                out[i] = x > T(0) ? x : T(0); // reference::relu
            else
                out[i] = x;
        }
    }

    template <typename TO>
    __device__ __forceinline__ TO convert_from_f(double v, bool from_f32)
    {
        return static_cast<TO>(v);
    }

    template <typename TI, typename TO>
    __global__ __launch_bounds__(256) void convert_kernel(const TI* in, TO* out, int64_t n)
    {
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < n; i += step)
        {
            TI x = in[i];
            if (std::is_floating_point<TI>::value && std::is_integral<TO>::value)
            {
                // x86: cvttss2si / cvttsd2si to 32 bits, then the low bits
                double d = static_cast<double>(x);
                int32_t t = (!(d < 2147483648.0) || d <= -2147483649.0) ? INT32_MIN : static_cast<int32_t>(d);
                out[i] = static_cast<TO>(t);
            }
            else
                out[i] = static_cast<TO>(x);
        }
    }

    struct BroadcastInfo
    {
        int32_t rank;
        uint32_t axes_mask;
        int64_t shape[HIPQ_MAX_RANK];
    };

    template <typename T>
    __global__ __launch_bounds__(256) void broadcast_kernel(const T* in, T* out, int64_t n, BroadcastInfo bi)
    {
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < n; i += step)
        {
            int64_t r = i, coord[HIPQ_MAX_RANK];
            for (int a = bi.rank - 1; a >= 0; --a)
            {
                coord[a] = r % bi.shape[a];
                r /= bi.shape[a];
            }
            int64_t j = 0;
            for (int a = 0; a < bi.rank; ++a)
                if (!(bi.axes_mask & (1u << a)))
                    j = j * bi.shape[a] + coord[a];
            out[i] = in[j];
        }
    }

    // out[c] = in[lower + c * stride] along every axis (src/ngraph/runtime/reference/slice.hpp:30-66)
    struct SliceInfo
    {
        int32_t rank;
        int64_t out_shape[HIPQ_MAX_RANK];
        int64_t in_step[HIPQ_MAX_RANK]; // elements of `in` one output step along the axis skips
        int64_t in_first;               // element of `in` at output coordinate 0
    };

    template <typename T>
    __global__ __launch_bounds__(256) void slice_kernel(const T* in, T* out, int64_t n, SliceInfo si)
    {
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < n; i += step)
        {
            int64_t r = i, j = si.in_first;
            for (int a = si.rank - 1; a >= 0; --a)
            {
                j += (r % si.out_shape[a]) * si.in_step[a];
                r /= si.out_shape[a];
            }
            out[i] = in[j];
        }
    }

    struct PermuteInfo
    {
        int32_t rank;
        int64_t out_shape[HIPQ_MAX_RANK];
        int64_t in_stride[HIPQ_MAX_RANK]; // stride in the input of output axis i
    };

    template <typename T>
    __global__ __launch_bounds__(256) void permute_kernel(const T* in, T* out, int64_t n, PermuteInfo pi)
    {
        int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
        for (; i < n; i += step)
        {
            int64_t r = i, j = 0;
            for (int a = pi.rank - 1; a >= 0; --a)
            {
                j += (r % pi.out_shape[a]) * pi.in_stride[a];
                r /= pi.out_shape[a];
            }
            out[i] = in[j];
        }
    }

    // the same with 32-bit index arithmetic (tensors below 2^31 elements) on 16-byte pieces: for orders
    // that keep the innermost axis, whose rows are whole pieces (splitting and merging attention heads)
    struct PermuteInfo32
    {
        int32_t rank;
        uint32_t out_shape[HIPQ_MAX_RANK];
        uint32_t in_stride[HIPQ_MAX_RANK];
    };

    __global__ __launch_bounds__(256) void permute_rows16_kernel(const uint4* __restrict__ in, uint4* __restrict__ out, uint32_t n, PermuteInfo32 pi)
    {
        const uint32_t i = blockIdx.x * 256u + threadIdx.x;
        if (i >= n)
            return;
        uint32_t r = i, j = 0;
        for (int a = pi.rank - 1; a >= 0; --a)
        {
            const uint32_t q = r / pi.out_shape[a];
            j += (r - q * pi.out_shape[a]) * pi.in_stride[a];
            r = q;
        }
        out[i] = in[j];
    }

    // 16 bytes per lane for the element types networks move in bulk: the same scalar expression per
    // element, on registers
    template <typename T, int OP>
    __global__ __launch_bounds__(256) void binary_vec_kernel(const uint4* __restrict__ a, const uint4* __restrict__ b, uint4* __restrict__ out, int64_t vecs)
    {
        constexpr int V = 16 / sizeof(T);
        union Pack
        {
            uint4 q;
            T e[V];
        };
        int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * 256;
        for (; i < vecs; i += step)
        {
            Pack x, y, r;
            x.q = a[i];
            y.q = b[i];
#pragma unroll
            for (int j = 0; j < V; ++j)
            {
                if (sizeof(T) == 1 && (OP == HIPQ_OP_DIVIDE || OP == HIPQ_OP_DIVIDE_FLOOR) && y.e[j] == 0)
                    r.e[j] = 0;
                else
                    r.e[j] = binary_apply<T>(OP, x.e[j], y.e[j]);
            }
            out[i] = r.q;
        }
    }

    template <typename T, int OP>
    __global__ __launch_bounds__(256) void unary_vec_kernel(const uint4* __restrict__ in, uint4* __restrict__ out, int64_t vecs)
    {
        constexpr int V = 16 / sizeof(T);
        union Pack
        {
            uint4 q;
            T e[V];
        };
        int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
        const int64_t step = static_cast<int64_t>(gridDim.x) * 256;
        for (; i < vecs; i += step)
        {
            Pack x;
            x.q = in[i];
            if (OP != HIPQ_OP_COPY)
            {
#pragma unroll
                for (int j = 0; j < V; ++j)
                {
                    const T v = x.e[j];
                    x.e[j] = OP == HIPQ_OP_ABS ? (v < T(0) ? static_cast<T>(-v) : v) : (v > T(0) ? v : T(0));
                }
            }
            out[i] = x.q;
        }
    }

    static unsigned blocks_for(int64_t n)
    {
        int64_t b = (n + 255) / 256;
        return static_cast<unsigned>(b < 1 ? 1 : (b > 65536 ? 65536 : b));
    }
}

using namespace hipq;

extern "C" {

int hipq_binary(int32_t op, int32_t dtype, const void* a, int64_t an, const void* b, int64_t bn, void* out, int64_t n, void* stream)
{
    HIPQ_REQUIRE(op >= HIPQ_OP_ADD && op <= HIPQ_OP_DIVIDE_FLOOR, "binary op %d unknown", op);
    HIPQ_REQUIRE(n >= 0 && (an == n || an == 1) && (bn == n || bn == 1), "operand counts must be the output count or 1");
    if (n == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(a && b && out, "null tensor pointer");
    hipStream_t s = as_stream(stream);
    // bulk tensors: whole 16-byte groups through the vector kernel, the remainder through the scalar one
    const size_t esz = dtype_size(dtype);
    if (an == n && bn == n && dtype != HIPQ_F64 && n * static_cast<int64_t>(esz) >= 4096 &&
        (reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(out)) % 16 == 0)
    {
        const int64_t per = 16 / static_cast<int64_t>(esz), vecs = n / per;
        const unsigned grid = blocks_for(vecs);
#define VEC_B(T, OP)                                                                               \
    case OP:                                                                                       \
        binary_vec_kernel<T, OP><<<grid, 256, 0, s>>>(static_cast<const uint4*>(a), static_cast<const uint4*>(b), static_cast<uint4*>(out), vecs); \
        break;
#define VEC_B_ALL(T)                                                                               \
    switch (op)                                                                                    \
    {                                                                                              \
        VEC_B(T, HIPQ_OP_ADD) VEC_B(T, HIPQ_OP_SUBTRACT) VEC_B(T, HIPQ_OP_MULTIPLY) VEC_B(T, HIPQ_OP_DIVIDE) VEC_B(T, HIPQ_OP_MAXIMUM)          \
            VEC_B(T, HIPQ_OP_MINIMUM) VEC_B(T, HIPQ_OP_DIVIDE_FLOOR)                               \
    }
        switch (dtype)
        {
        case HIPQ_U8: VEC_B_ALL(uint8_t) break;
        case HIPQ_I8: VEC_B_ALL(int8_t) break;
        case HIPQ_I32: VEC_B_ALL(int32_t) break;
        case HIPQ_F32: VEC_B_ALL(float) break;
        default: return fail(HIPQ_ERR_UNSUPPORTED, "element type %d", dtype);
        }
#undef VEC_B_ALL
#undef VEC_B
        int rc = check_launch("binary_vec");
        const int64_t done = vecs * per;
        if (rc || done == n)
            return rc;
        return hipq_binary(op, dtype, static_cast<const char*>(a) + done * esz, n - done, static_cast<const char*>(b) + done * esz, n - done,
                           static_cast<char*>(out) + done * esz, n - done, stream);
    }
#define LAUNCH_B(T) binary_kernel<T><<<blocks_for(n), 256, 0, s>>>(op, static_cast<const T*>(a), an, static_cast<const T*>(b), bn, static_cast<T*>(out), n)
    switch (dtype)
    {
    case HIPQ_U8: LAUNCH_B(uint8_t); break;
    case HIPQ_I8: LAUNCH_B(int8_t); break;
    case HIPQ_I32: LAUNCH_B(int32_t); break;
    case HIPQ_F32: LAUNCH_B(float); break;
    case HIPQ_F64: LAUNCH_B(double); break;
    default: return fail(HIPQ_ERR_UNSUPPORTED, "element type %d", dtype);
    }
#undef LAUNCH_B
    return check_launch("binary");
}

int hipq_unary(int32_t op, int32_t dtype, const void* in, void* out, int64_t n, void* stream)
{
    HIPQ_REQUIRE(op >= HIPQ_OP_ABS && op <= HIPQ_OP_COPY, "unary op %d unknown", op);
    HIPQ_REQUIRE(n >= 0, "negative count");
    if (n == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && out, "null tensor pointer");
    hipStream_t s = as_stream(stream);
    const size_t esz = dtype_size(dtype);
    if (dtype != HIPQ_F64 && n * static_cast<int64_t>(esz) >= 4096 && (reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) % 16 == 0)
    {
        const int64_t per = 16 / static_cast<int64_t>(esz), vecs = n / per;
        const unsigned grid = blocks_for(vecs);
#define VEC_U(T, OP)                                                                               \
    case OP: unary_vec_kernel<T, OP><<<grid, 256, 0, s>>>(static_cast<const uint4*>(in), static_cast<uint4*>(out), vecs); break;
#define VEC_U_ALL(T)                                                                               \
    switch (op)                                                                                    \
    {                                                                                              \
        VEC_U(T, HIPQ_OP_ABS) VEC_U(T, HIPQ_OP_RELU) VEC_U(T, HIPQ_OP_COPY)                        \
    }
        switch (dtype)
        {
        case HIPQ_U8: VEC_U_ALL(uint8_t) break;
        case HIPQ_I8: VEC_U_ALL(int8_t) break;
        case HIPQ_I32: VEC_U_ALL(int32_t) break;
        case HIPQ_F32: VEC_U_ALL(float) break;
        default: return fail(HIPQ_ERR_UNSUPPORTED, "element type %d", dtype);
        }
#undef VEC_U_ALL
#undef VEC_U
        int rc = check_launch("unary_vec");
        const int64_t done = vecs * per;
        if (rc || done == n)
            return rc;
        return hipq_unary(op, dtype, static_cast<const char*>(in) + done * esz, static_cast<char*>(out) + done * esz, n - done, stream);
    }
#define LAUNCH_U(T) unary_kernel<T><<<blocks_for(n), 256, 0, s>>>(op, static_cast<const T*>(in), static_cast<T*>(out), n)
    switch (dtype)
    {
    case HIPQ_U8: LAUNCH_U(uint8_t); break;
    case HIPQ_I8: LAUNCH_U(int8_t); break;
    case HIPQ_I32: LAUNCH_U(int32_t); break;
    case HIPQ_F32: LAUNCH_U(float); break;
    case HIPQ_F64: LAUNCH_U(double); break;
    default: return fail(HIPQ_ERR_UNSUPPORTED, "element type %d", dtype);
    }
#undef LAUNCH_U
    return check_launch("unary");
}

int hipq_convert(int32_t in_t, int32_t out_t, const void* in, void* out, int64_t n, void* stream)
{
    HIPQ_REQUIRE(n >= 0, "negative count");
    if (n == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && out, "null tensor pointer");
    // between the two 8-bit types, and within one type, static_cast keeps the bits (the reference's CPU
    // backend aliases the buffers for it, src/ngraph/runtime/cpu/pass/cpu_assignment.cpp:983-997)
    if (in_t == out_t || ((in_t == HIPQ_U8 || in_t == HIPQ_I8) && (out_t == HIPQ_U8 || out_t == HIPQ_I8)))
        return hipq_unary(HIPQ_OP_COPY, out_t, in, out, n, stream);
    hipStream_t s = as_stream(stream);
#define LAUNCH_C(TI, TO) convert_kernel<TI, TO><<<blocks_for(n), 256, 0, s>>>(static_cast<const TI*>(in), static_cast<TO*>(out), n)
#define CONVERT_TO(TI)                                                                             \
    switch (out_t)                                                                                 \
    {                                                                                              \
    case HIPQ_U8: LAUNCH_C(TI, uint8_t); break;                                                    \
    case HIPQ_I8: LAUNCH_C(TI, int8_t); break;                                                     \
    case HIPQ_I32: LAUNCH_C(TI, int32_t); break;                                                   \
    case HIPQ_F32: LAUNCH_C(TI, float); break;                                                     \
    case HIPQ_F64: LAUNCH_C(TI, double); break;                                                    \
    default: return fail(HIPQ_ERR_UNSUPPORTED, "element type %d", out_t);                          \
    }
    switch (in_t)
    {
    case HIPQ_U8: CONVERT_TO(uint8_t); break;
    case HIPQ_I8: CONVERT_TO(int8_t); break;
    case HIPQ_I32: CONVERT_TO(int32_t); break;
    case HIPQ_F32: CONVERT_TO(float); break;
    case HIPQ_F64: CONVERT_TO(double); break;
    default: return fail(HIPQ_ERR_UNSUPPORTED, "element type %d", in_t);
    }
#undef CONVERT_TO
#undef LAUNCH_C
    return check_launch("convert");
}

int hipq_broadcast(int32_t elem_bytes, const void* in, void* out, int32_t rank, const int64_t* shape, uint32_t axes_mask, void* stream)
{
    HIPQ_REQUIRE(rank >= 0 && rank <= HIPQ_MAX_RANK, "rank %d out of range", rank);
    HIPQ_REQUIRE(rank == 0 || shape, "shape is null");
    BroadcastInfo bi;
    bi.rank = rank;
    bi.axes_mask = axes_mask;
    int64_t n = 1;
    for (int i = 0; i < HIPQ_MAX_RANK; ++i)
    {
        bi.shape[i] = i < rank ? shape[i] : 1;
        HIPQ_REQUIRE(bi.shape[i] >= 0, "negative extent");
        n *= bi.shape[i];
    }
    if (n == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && out, "null tensor pointer");
    hipStream_t s = as_stream(stream);
    switch (elem_bytes)
    {
    case 1: broadcast_kernel<uint8_t><<<blocks_for(n), 256, 0, s>>>(static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), n, bi); break;
    case 4: broadcast_kernel<uint32_t><<<blocks_for(n), 256, 0, s>>>(static_cast<const uint32_t*>(in), static_cast<uint32_t*>(out), n, bi); break;
    case 8: broadcast_kernel<uint64_t><<<blocks_for(n), 256, 0, s>>>(static_cast<const uint64_t*>(in), static_cast<uint64_t*>(out), n, bi); break;
    default: return fail(HIPQ_ERR_UNSUPPORTED, "%d-byte elements", elem_bytes);
    }
    return check_launch("broadcast");
}

int hipq_slice(int32_t elem_bytes, const void* in, void* out, int32_t rank, const int64_t* in_shape, const int64_t* lower, const int64_t* upper, const int64_t* strides, void* stream)
{
    HIPQ_REQUIRE(rank >= 0 && rank <= HIPQ_MAX_RANK, "rank %d out of range", rank);
    HIPQ_REQUIRE(rank == 0 || (in_shape && lower && upper && strides), "shape, bounds or strides are null");
    SliceInfo si;
    si.rank = rank;
    si.in_first = 0;
    int64_t n = 1, in_stride = 1;
    for (int i = 0; i < HIPQ_MAX_RANK; ++i)
    {
        si.out_shape[i] = 1;
        si.in_step[i] = 0;
    }
    for (int i = rank - 1; i >= 0; --i)
    {
        HIPQ_REQUIRE(in_shape[i] >= 0 && strides[i] >= 1, "negative extent or non-positive stride on axis %d", i);
        HIPQ_REQUIRE(lower[i] >= 0 && lower[i] <= upper[i] && upper[i] <= in_shape[i], "bounds [%lld, %lld) outside axis %d of extent %lld", static_cast<long long>(lower[i]),
                     static_cast<long long>(upper[i]), i, static_cast<long long>(in_shape[i]));
        si.out_shape[i] = (upper[i] - lower[i] + strides[i] - 1) / strides[i]; // ceil
        si.in_step[i] = in_stride * strides[i];
        si.in_first += in_stride * lower[i];
        n *= si.out_shape[i];
        in_stride *= in_shape[i];
    }
    if (n == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && out, "null tensor pointer");
    hipStream_t s = as_stream(stream);
    switch (elem_bytes)
    {
    case 1: slice_kernel<uint8_t><<<blocks_for(n), 256, 0, s>>>(static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), n, si); break;
    case 4: slice_kernel<uint32_t><<<blocks_for(n), 256, 0, s>>>(static_cast<const uint32_t*>(in), static_cast<uint32_t*>(out), n, si); break;
    case 8: slice_kernel<uint64_t><<<blocks_for(n), 256, 0, s>>>(static_cast<const uint64_t*>(in), static_cast<uint64_t*>(out), n, si); break;
    default: return fail(HIPQ_ERR_UNSUPPORTED, "%d-byte elements", elem_bytes);
    }
    return check_launch("slice");
}

int hipq_permute(int32_t elem_bytes, const void* in, void* out, int32_t rank, const int64_t* in_shape, const int32_t* order, void* stream)
{
    HIPQ_REQUIRE(rank >= 0 && rank <= HIPQ_MAX_RANK, "rank %d out of range", rank);
    HIPQ_REQUIRE(rank == 0 || (in_shape && order), "shape or order is null");
    int64_t stride[HIPQ_MAX_RANK];
    int64_t n = 1;
    for (int i = rank - 1; i >= 0; --i)
    {
        HIPQ_REQUIRE(in_shape[i] >= 0, "negative extent");
        stride[i] = n;
        n *= in_shape[i];
    }
    PermuteInfo pi;
    pi.rank = rank;
    uint32_t seen = 0;
    for (int i = 0; i < HIPQ_MAX_RANK; ++i)
    {
        pi.out_shape[i] = 1;
        pi.in_stride[i] = 0;
    }
    for (int i = 0; i < rank; ++i)
    {
        HIPQ_REQUIRE(order[i] >= 0 && order[i] < rank && !(seen & (1u << order[i])), "order is not a permutation");
        seen |= 1u << order[i];
        pi.out_shape[i] = in_shape[order[i]];
        pi.in_stride[i] = stride[order[i]];
    }
    if (n == 0)
        return HIPQ_OK;
    HIPQ_REQUIRE(in && out, "null tensor pointer");
    hipStream_t s = as_stream(stream);
    if (elem_bytes == 1 || elem_bytes == 4)
    {
        // order = (0..b-1 | m..rank-1 | b..m-1) is a batched 2-D transpose [B][R][C] -> [B][C][R]: the
        // NCHW <-> NHWC changes are of this kind
        int lead = 0;
        while (lead < rank && order[lead] == lead)
            ++lead;
        if (lead == rank)
            return hipq_memcpy_d2d(out, in, static_cast<size_t>(n) * elem_bytes, stream);
        const int m = order[lead];
        bool two_blocks = m > lead;
        for (int i = lead; two_blocks && i < rank; ++i)
            two_blocks = order[i] == (i - lead < rank - m ? m + (i - lead) : lead + (i - lead - (rank - m)));
        if (two_blocks)
        {
            int64_t B = 1, R = 1, Cc = 1;
            for (int i = 0; i < lead; ++i)
                B *= in_shape[i];
            for (int i = lead; i < m; ++i)
                R *= in_shape[i];
            for (int i = m; i < rank; ++i)
                Cc *= in_shape[i];
            if (R < 65535 * 64 && Cc < (1ll << 31) && B < 65536)
                return launch_transpose(in, out, B, R, Cc, elem_bytes, s);
        }
    }
    // the innermost axis stays innermost and its rows are whole 16-byte pieces: move pieces
    if (rank >= 2 && order[rank - 1] == rank - 1 && (in_shape[rank - 1] * elem_bytes) % 16 == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 &&
        n * elem_bytes / 16 < (1ll << 31))
    {
        const int64_t per = 16 / elem_bytes; // elements per piece
        PermuteInfo32 p32;
        p32.rank = rank;
        for (int i = 0; i < HIPQ_MAX_RANK; ++i)
        {
            p32.out_shape[i] = 1;
            p32.in_stride[i] = 0;
        }
        for (int i = 0; i < rank; ++i)
        {
            p32.out_shape[i] = static_cast<uint32_t>(i == rank - 1 ? pi.out_shape[i] / per : pi.out_shape[i]);
            p32.in_stride[i] = static_cast<uint32_t>(i == rank - 1 ? 1 : pi.in_stride[i] / per);
        }
        const uint32_t pieces = static_cast<uint32_t>(n / per);
        permute_rows16_kernel<<<(pieces + 255) / 256, 256, 0, s>>>(static_cast<const uint4*>(in), static_cast<uint4*>(out), pieces, p32);
        return check_launch("permute_rows16");
    }
    switch (elem_bytes)
    {
    case 1: permute_kernel<uint8_t><<<blocks_for(n), 256, 0, s>>>(static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), n, pi); break;
    case 4: permute_kernel<uint32_t><<<blocks_for(n), 256, 0, s>>>(static_cast<const uint32_t*>(in), static_cast<uint32_t*>(out), n, pi); break;
    case 8: permute_kernel<uint64_t><<<blocks_for(n), 256, 0, s>>>(static_cast<const uint64_t*>(in), static_cast<uint64_t*>(out), n, pi); break;
    default: return fail(HIPQ_ERR_UNSUPPORTED, "%d-byte elements", elem_bytes);
    }
    return check_launch("permute");
}
}
