// A measurement aid, not part of the path: how fast the matrix cores run when nothing else limits
// them.  Every wavefront of a full-chip launch issues one dependent chain of v_mfma_i32_32x32x32_i8
// on operands it holds in registers -- no memory traffic, no LDS, no other instructions -- so the
// rate reached is the ceiling any int8 kernel has on this device for operands of that kind.  The
// ceiling depends on the operand bytes (the chip lowers its clock under the switching activity of
// dense data): bench.py reports it for all-zero and for random bytes next to the convolution's rate.
#include "hipq_common.h"

namespace hipq
{
    typedef int pv4i __attribute__((ext_vector_type(4)));
    typedef int pv16i __attribute__((ext_vector_type(16)));

    // ops: 8 operand sets of 64 lanes x 16 bytes (4 for the A side, 4 for the B side)
    __global__ __launch_bounds__(256) void probe_mfma_i8_kernel(const pv4i* __restrict__ ops, int* __restrict__ sink, int iters)
    {
        pv16i acc[2];
        for (int i = 0; i < 2; ++i)
            for (int r = 0; r < 16; ++r)
                acc[i][r] = i;
        pv4i a[4], b[4];
        for (int i = 0; i < 4; ++i)
        {
            a[i] = ops[(i * 2) * 64 + (threadIdx.x & 63)];
            b[i] = ops[(i * 2 + 1) * 64 + (threadIdx.x & 63)];
        }
        for (int it = 0; it < iters; ++it)
        {
#pragma unroll
            for (int i = 0; i < 64; ++i)
                acc[i & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i & 3], b[(i >> 2) & 3], acc[i & 1], 0, 0, 0);
        }
        int s = 0;
        for (int i = 0; i < 2; ++i)
            for (int r = 0; r < 16; ++r)
                s += acc[i][r];
        sink[blockIdx.x * 256 + threadIdx.x] = s;
    }
}

using namespace hipq;

extern "C" {

int hipq_probe_mfma_i8(const void* operands_8k, void* sink, int32_t workgroups, int32_t iters, void* stream)
{
    HIPQ_REQUIRE(operands_8k && sink, "null pointer");
    HIPQ_REQUIRE(workgroups > 0 && workgroups <= 65535 && iters > 0 && iters <= 100000, "workgroups / iterations out of range");
    HIPQ_REQUIRE((reinterpret_cast<uintptr_t>(operands_8k) & 15) == 0, "operands must be 16-byte aligned");
    probe_mfma_i8_kernel<<<static_cast<unsigned>(workgroups), 256, 0, as_stream(stream)>>>(static_cast<const pv4i*>(operands_8k), static_cast<int*>(sink), iters);
    return check_launch("probe_mfma_i8");
}
}
