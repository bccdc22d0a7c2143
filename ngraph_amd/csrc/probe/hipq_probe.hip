// Measurement aids (libhipq_probe.so): device ceilings that the kernels of libhipq.so are judged
// against.  Nothing here is on the product path; see hipq_probe.h.
//   * probe_mfma_i8_kernel: how fast the matrix cores run when nothing else limits them.  Every
//     wavefront of a full-chip launch issues one dependent chain of v_mfma_i32_32x32x32_i8 on
//     operands it holds in registers -- no memory traffic, no LDS, no other instructions.  The rate
//     depends on the operand bytes (the chip lowers its clock under the switching activity of
//     dense data).
//   * probe_intake_kernel: bytes a second a compute unit takes in from L2 / HBM, by load shape
//     and destination (registers or LDS).
//   * probe_atomic_tiles_kernel: integer atomic adds of whole accumulator tiles into L2.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>

#include "../hipq_index_div.h"
#include "hipq_probe.h"

namespace
{
    thread_local char t_error[256] = "";

    int fail(const char* fmt, ...)
    {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(t_error, sizeof(t_error), fmt, ap);
        va_end(ap);
        return 1;
    }

    int check_launch(const char* what)
    {
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? 0 : fail("launch of %s failed: %s", what, hipGetErrorString(e));
    }

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

    // Do matrix and vector instructions share a SIMD's time?  MODE 0: every wavefront issues 16 MFMAs
    // an iteration with V independent v_fma_f32 behind each (the compiler is held to that order);
    // 1: the MFMAs alone; 2: the vector instructions alone; 3: a workgroup of eight wavefronts, two a
    // SIMD, of which the first four issue only the MFMAs and the last four only the vector instructions;
    // 4: as 0 with the accumulators named in the accumulation half of the register file.
    template <int V, int MODE>
    __global__ __launch_bounds__(512) void probe_coissue_kernel(const pv4i* __restrict__ ops, int* __restrict__ sink, int iters)
    {
        pv16i acc[2];
        for (int i = 0; i < 2; ++i)
            for (int r = 0; r < 16; ++r)
                acc[i][r] = i;
        const pv4i a = ops[threadIdx.x & 63], b = ops[64 + (threadIdx.x & 63)];
        float x[8];
        for (int k = 0; k < 8; ++k)
            x[k] = static_cast<float>(a[k & 3] & 0xFF) * 1e-3f;
        const float c = 0.999f + static_cast<float>(b[0] & 1) * 1e-4f, d = static_cast<float>(b[1] & 3) * 1e-3f;
        const bool matrix = MODE == 0 || MODE == 1 || (MODE == 3 && (threadIdx.x >> 8) == 0);
        const bool vector = MODE == 0 || MODE == 2 || (MODE == 3 && (threadIdx.x >> 8) == 1);
        for (int it = 0; it < iters; ++it)
        {
            if (MODE == 4)
            {
                // as mode 0 with the accumulators in the accumulation registers (AGPRs): the MFMA's 16
                // registers of input and output then do not pass through the vector register file's ports
#pragma unroll
                for (int i = 0; i < 16; ++i)
                {
                    if (i & 1)
                        asm volatile("v_mfma_i32_32x32x32_i8 a[16:31], %0, %1, a[16:31]" ::"v"(a), "v"(b)
                                     : "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31");
                    else
                        asm volatile("v_mfma_i32_32x32x32_i8 a[0:15], %0, %1, a[0:15]" ::"v"(a), "v"(b)
                                     : "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15");
#pragma unroll
                    for (int v = 0; v < V; ++v)
                        asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[v & 7]) : "v"(c), "v"(d));
                }
            }
            else if (MODE == 0)
            {
#pragma unroll
                for (int i = 0; i < 16; ++i)
                {
                    acc[i & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[i & 1], 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < V; ++v)
                        x[v & 7] = __builtin_fmaf(x[v & 7], c, d);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, V, 0);
                }
            }
            else
            {
                if (matrix) // uniform per wavefront
                {
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        acc[i & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[i & 1], 0, 0, 0);
                }
                if (vector)
                {
#pragma unroll
                    for (int i = 0; i < 16 * V; ++i)
                        x[i & 7] = __builtin_fmaf(x[i & 7], c, d);
                }
            }
        }
        int s = 0;
        for (int i = 0; i < 2; ++i)
            for (int r = 0; r < 16; ++r)
                s += acc[i][r];
        float f = 0.0f;
        for (int k = 0; k < 8; ++k)
            f += x[k];
        sink[blockIdx.x * 512 + threadIdx.x] = s + static_cast<int>(f);
    }

    constexpr int kIntakeLoads = 8;       // 16-byte loads a lane and step
    constexpr int kIntakeStepBytes = 32768; // 4 wavefronts x 8 instructions x 1 KiB

    // byte offset (before wrapping) of load u of step `step` for this lane
    template <int SHAPE>
    __device__ __forceinline__ uint32_t intake_offset(uint32_t base, uint32_t step, int wave, int lane, int u)
    {
        if (SHAPE == 0) // 1 KiB contiguous an instruction, a step is 32 KiB contiguous
            return base + step * kIntakeStepBytes + static_cast<uint32_t>((wave * kIntakeLoads + u) * 1024 + lane * 16);
        // row pieces out of rows kPitch bytes apart: a workgroup's step is a block of 256 (128-byte
        // pieces), 512 (64-byte pieces) or 2048 (16-byte pieces: every lane in a line of its own,
        // what a wavefront reading MFMA fragments out of a row-major matrix does) rows at one column;
        // the steps sweep the columns of a row, then the block moves on by its rows
        constexpr int PIECE = SHAPE == 1 ? 128 : SHAPE == 2 ? 64 : 16;
        constexpr uint32_t kPitch = SHAPE == 3 ? 1024u : 4096u;
        constexpr int LANES = PIECE / 16;      // lanes a row piece
        constexpr int ROWS = 64 / LANES;       // rows an instruction
        constexpr int BLOCK_ROWS = 4 * kIntakeLoads * ROWS;
        constexpr int SWEEP = kPitch / PIECE;  // steps until the columns wrap (a power of two)
        const uint32_t row = static_cast<uint32_t>((wave * kIntakeLoads + u) * ROWS + lane / LANES);
        const uint32_t col = (step & (SWEEP - 1)) * PIECE + static_cast<uint32_t>(lane % LANES) * 16;
        return base + (step / SWEEP) * (BLOCK_ROWS * kPitch) + row * kPitch + col;
    }

    template <int SHAPE, bool TO_LDS>
    __global__ __launch_bounds__(256) void probe_intake_kernel(const uint8_t* __restrict__ buf, uint32_t buf_bytes, uint32_t window_mask, uint32_t spread_bytes, int steps, int* __restrict__ sink)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
        const int lane = threadIdx.x & 63;
        const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(buf), 0, static_cast<int>(buf_bytes), 0x00020000);
        // spread: every workgroup has a region of its own; else a start of its own inside the shared
        // window (4 KiB-aligned, scattered), so that the compute units do not walk the same L2
        // channel in step
        const uint32_t base = spread_bytes == 1u ? 0u : spread_bytes ? static_cast<uint32_t>(blockIdx.x) * spread_bytes : (static_cast<uint32_t>(blockIdx.x) * 0x9E3779B1u) & ~0xFFFu;
        pv4i acc = {0, 0, 0, 0};
        if (TO_LDS)
        {
            // wavefront w lands its 8 KiB of a step at lds + w * 8 KiB (the same place every step: nothing reads it)
            const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + static_cast<uint32_t>(wave) * 8192u;
            for (int s = 0; s < steps; ++s)
            {
#pragma unroll
                for (int u = 0; u < kIntakeLoads; ++u)
                {
                    const uint32_t off = intake_offset<SHAPE>(base, static_cast<uint32_t>(s), wave, lane, u) & window_mask;
                    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_base + static_cast<uint32_t>(u) * 1024u), "v"(off), "s"(rs) : "memory");
                }
                // the step before this one has landed; this one stays in flight
                asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            acc[0] = *reinterpret_cast<const int*>(lds + threadIdx.x * 4);
        }
        else
        {
            pv4i cur[kIntakeLoads], nxt[kIntakeLoads];
#pragma unroll
            for (int u = 0; u < kIntakeLoads; ++u)
                cur[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, intake_offset<SHAPE>(base, 0u, wave, lane, u) & window_mask, 0, 0);
            for (int s = 1; s <= steps; ++s)
            {
                // (one step past the end: a harmless re-read inside the window)
#pragma unroll
                for (int u = 0; u < kIntakeLoads; ++u)
                    nxt[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, intake_offset<SHAPE>(base, static_cast<uint32_t>(s), wave, lane, u) & window_mask, 0, 0);
#pragma unroll
                for (int u = 0; u < kIntakeLoads; ++u)
                    acc ^= cur[u];
#pragma unroll
                for (int u = 0; u < kIntakeLoads; ++u)
                    cur[u] = nxt[u];
            }
        }
        sink[blockIdx.x * 256 + threadIdx.x] = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    }

    // a kernel that does nothing but exist: `touch` != 0 makes lane 0 of every workgroup write one word
    __global__ __launch_bounds__(256) void probe_empty_kernel(int* __restrict__ sink, int touch)
    {
        if (touch && threadIdx.x == 0)
            sink[blockIdx.x] = touch;
    }

    // a workgroup of 256 lanes holds a 128 x 128 int32 tile as 64 values a lane; value j of lane t is
    // element j * 256 + t of the tile (a wavefront instruction covers 256 contiguous bytes)
    __global__ __launch_bounds__(256) void probe_atomic_tiles_kernel(int* __restrict__ dst, int share, int same_die, int rounds, int groups)
    {
        const int wg = static_cast<int>(blockIdx.x);
        // same die: workgroups g, g + 8, ... (ids congruent modulo 8) share; else consecutive ids share
        int group;
        if (same_die)
        {
            const int die = wg & 7, k = wg >> 3; // k-th workgroup of its die
            group = (k / share) * 8 + die;
        }
        else
            group = wg / share;
        if (group >= groups)
            return;
        for (int r = 0; r < rounds; ++r)
        {
            int* tile = dst + (static_cast<size_t>(group) * rounds + r) * 16384;
#pragma unroll 16
            for (int j = 0; j < 64; ++j)
                __hip_atomic_fetch_add(tile + j * 256 + threadIdx.x, wg + j + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

extern "C" {

const char* hipq_probe_last_error(void)
{
    return t_error;
}

int hipq_probe_mfma_i8(const void* operands_8k, void* sink, int32_t workgroups, int32_t iters, void* stream)
{
    if (!operands_8k || !sink)
        return fail("null pointer");
    if (workgroups <= 0 || workgroups > 65535 || iters <= 0 || iters > 100000)
        return fail("workgroups / iterations out of range");
    if (reinterpret_cast<uintptr_t>(operands_8k) & 15)
        return fail("operands must be 16-byte aligned");
    probe_mfma_i8_kernel<<<static_cast<unsigned>(workgroups), 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const pv4i*>(operands_8k), static_cast<int*>(sink), iters);
    return check_launch("probe_mfma_i8");
}

int hipq_probe_coissue(const void* operands_2k, void* sink, int32_t workgroups, int32_t iters, int32_t vector_per_mfma, int32_t mode, void* stream)
{
    if (!operands_2k || !sink)
        return fail("null pointer");
    if (workgroups <= 0 || workgroups > 65535 || iters <= 0 || iters > 100000)
        return fail("workgroups / iterations out of range");
    if (mode < 0 || mode > 4 || (vector_per_mfma != 4 && vector_per_mfma != 8 && vector_per_mfma != 16))
        return fail("mode 0..3, 4, 8 or 16 vector instructions an MFMA");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const pv4i* ops = static_cast<const pv4i*>(operands_2k);
    int* out = static_cast<int*>(sink);
    const unsigned grid = static_cast<unsigned>(workgroups);
#define COISSUE(V)                                                        \
    switch (mode)                                                         \
    {                                                                     \
    case 0: probe_coissue_kernel<V, 0><<<grid, 512, 0, s>>>(ops, out, iters); break; \
    case 1: probe_coissue_kernel<V, 1><<<grid, 512, 0, s>>>(ops, out, iters); break; \
    case 2: probe_coissue_kernel<V, 2><<<grid, 512, 0, s>>>(ops, out, iters); break; \
    case 3: probe_coissue_kernel<V, 3><<<grid, 512, 0, s>>>(ops, out, iters); break; \
    default: probe_coissue_kernel<V, 4><<<grid, 512, 0, s>>>(ops, out, iters); break; \
    }
    if (vector_per_mfma == 4)
    {
        COISSUE(4)
    }
    else if (vector_per_mfma == 8)
    {
        COISSUE(8)
    }
    else
    {
        COISSUE(16)
    }
#undef COISSUE
    return check_launch("probe_coissue");
}

int hipq_probe_intake(const void* buf, size_t buf_bytes, size_t window_bytes, int32_t spread, int32_t shape, int32_t to_lds, int32_t workgroups, int32_t lds_bytes, int32_t steps,
                      void* sink, void* stream)
{
    if (!buf || !sink)
        return fail("null pointer");
    if (reinterpret_cast<uintptr_t>(buf) & 15)
        return fail("buffer must be 16-byte aligned");
    if (window_bytes < (1u << 20) || (window_bytes & (window_bytes - 1)) != 0 || window_bytes > buf_bytes || buf_bytes > 0xFFFFFFFFull)
        return fail("window must be a power of two of at least 1 MiB inside a buffer below 4 GiB");
    if (shape < 0 || shape > 3 || workgroups <= 0 || workgroups > 65535 || steps <= 0 || steps > (1 << 20))
        return fail("shape / workgroups / steps out of range");
    if (lds_bytes < (to_lds ? 32768 : 0) || lds_bytes > 160 * 1024)
        return fail("lds_bytes out of range (loads into LDS need 32 KiB)");
    const uint32_t mask = static_cast<uint32_t>(window_bytes - 1) & ~15u;
    const uint32_t spread_bytes = spread == 2 ? 1u : spread ? static_cast<uint32_t>(steps) * kIntakeStepBytes : 0u; // 2: every workgroup walks the same addresses in step
    hipStream_t s = static_cast<hipStream_t>(stream);
#define HIPQ_INTAKE(SHAPE, LDS)                                                                                                                              \
    do                                                                                                                                                       \
    {                                                                                                                                                        \
        auto k = probe_intake_kernel<SHAPE, LDS>;                                                                                                            \
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)                    \
            return fail("cannot raise the LDS limit");                                                                                                       \
        k<<<static_cast<unsigned>(workgroups), 256, static_cast<size_t>(lds_bytes), s>>>(static_cast<const uint8_t*>(buf), static_cast<uint32_t>(buf_bytes), mask, spread_bytes, steps, \
                                                                                          static_cast<int*>(sink));                                          \
    } while (0)
    if (to_lds)
    {
        if (shape == 0)
            HIPQ_INTAKE(0, true);
        else if (shape == 1)
            HIPQ_INTAKE(1, true);
        else if (shape == 2)
            HIPQ_INTAKE(2, true);
        else
            HIPQ_INTAKE(3, true);
    }
    else
    {
        if (shape == 0)
            HIPQ_INTAKE(0, false);
        else if (shape == 1)
            HIPQ_INTAKE(1, false);
        else if (shape == 2)
            HIPQ_INTAKE(2, false);
        else
            HIPQ_INTAKE(3, false);
    }
#undef HIPQ_INTAKE
    return check_launch("probe_intake");
}

int hipq_probe_atomic_tiles(void* dst, size_t dst_bytes, int32_t workgroups, int32_t share, int32_t same_die, int32_t rounds, void* stream)
{
    if (!dst)
        return fail("null pointer");
    if (workgroups <= 0 || workgroups > 65535 || share <= 0 || rounds <= 0 || rounds > 4096)
        return fail("workgroups / share / rounds out of range");
    if (workgroups % (same_die ? 8 * share : share) != 0)
        return fail("workgroups must be a multiple of %d", same_die ? 8 * share : share);
    const int groups = workgroups / share;
    if (static_cast<size_t>(groups) * static_cast<size_t>(rounds) * 65536 > dst_bytes)
        return fail("destination holds fewer than %d x %d tiles of 64 KiB", groups, rounds);
    probe_atomic_tiles_kernel<<<static_cast<unsigned>(workgroups), 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<int*>(dst), share, same_die, rounds, groups);
    return check_launch("probe_atomic_tiles");
}

int hipq_probe_empty_chain(void* sink, int32_t kernels, int32_t workgroups, int32_t touch, void* stream)
{
    if (!sink || kernels <= 0 || kernels > 4096 || workgroups <= 0 || workgroups > 65535)
        return fail("kernels / workgroups out of range");
    for (int i = 0; i < kernels; ++i)
        probe_empty_kernel<<<static_cast<unsigned>(workgroups), 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<int*>(sink), touch);
    return check_launch("probe_empty");
}

uint32_t hipq_debug_fastdiv(uint32_t n, uint32_t d)
{
    return hipq::fastdiv(n, hipq::make_fastdiv(d));
}
}
